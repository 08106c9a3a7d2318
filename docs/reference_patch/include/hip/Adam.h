// include/hip/Adam.h -- replaces include/cuda/Adam.h:49-90 (four cublasSscal/Saxpy, mulGpu, adamGpu and a
// fill per tensor) by one launch per tensor with the same per-element operation order.
#pragma once

#include "HipError.h"

namespace px {

template<>
inline void Adam<Device::HIP>::update(V& w, V& d, V& m, V& v, bool applyDecay)
{
    PX_HIP_CHECK(pxh_adam_update(w.size(), w.data(), d.data(), m.data(), v.data(), batch_, t_, lr_, beta1_, beta2_,
                                 epsilon_, decay_, applyDecay ? 1 : 0, nullptr));
}

}   // px
