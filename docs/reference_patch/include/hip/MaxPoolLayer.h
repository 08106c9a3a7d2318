// include/hip/MaxPoolLayer.h -- replaces include/cuda/MaxPoolLayer.h:23-54 (maxPoolForwardGpu / maxPoolBackwardGpu).
#pragma once

#include "HipError.h"

namespace px {

template<>
class MPExtras<Device::HIP>
{
protected:
    PxHipVectorT<int> indexes_;
};

template<>
inline void MaxPoolLayer<Device::HIP>::setup()
{
    indexes_ = PxHipVectorT<int>(this->batch() * this->outputs(), -1);
}

template<>
inline void MaxPoolLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    PX_HIP_CHECK(pxh_maxpool_forward(input.data(), this->output_.data(), indexes_.data(), this->batch(), this->channels(),
                                     this->height(), this->width(), this->outHeight(), this->outWidth(), kernel_, stride_,
                                     padding_, nullptr));
}

template<>
inline void MaxPoolLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    if (grad == nullptr) return;
    PX_HIP_CHECK(pxh_maxpool_backward(this->delta_.data(), indexes_.data(), grad->data(), this->batch(), this->channels(),
                                      this->height(), this->width(), this->outHeight(), this->outWidth(), kernel_,
                                      stride_, padding_, nullptr));
}

}   // px
