// Fused fp32 Adam step for one parameter tensor (reference: Adam<Device::CUDA>::update,
// include/cuda/Adam.h:49-90: seven cuBLAS / kernel passes; here one).
#pragma once

#include "Layer.h"

namespace px::hip {

class Adam
{
public:
    using V = FloatVector;

    Adam(hipStream_t stream, int batch, int t, float lr, float beta1, float beta2, float epsilon, float decay)
            : stream_(stream), batch_(batch), t_(t), lr_(lr), beta1_(beta1), beta2_(beta2), epsilon_(epsilon),
              decay_(decay)
    {
        PX_CHECK(batch > 0 && t > 0, "Adam needs batch > 0 and t > 0");
    }

    explicit Adam(const Context& c) : Adam(c.stream, c.updateBatch, c.timeStep, c.learningRate, c.adamBeta1,
                                           c.adamBeta2, c.adamEpsilon, c.decay) {}

    // w: parameters, d: accumulated update (consumed: zero afterwards), m / v: moments.
    void update(V& w, V& d, V& m, V& v, bool applyDecay) const
    {
        PX_CHECK(w.size() == d.size() && w.size() == m.size() && w.size() == v.size(),
                 "Adam: tensors of different sizes");
        PX_HIP_CHECK(pxh_adam_update(w.size(), w.data(), d.data(), m.data(), v.data(), batch_, t_, lr_, beta1_,
                                     beta2_, epsilon_, decay_, applyDecay ? 1 : 0, stream_));
    }

private:
    hipStream_t stream_;
    int batch_, t_;
    float lr_, beta1_, beta2_, epsilon_, decay_;
};

}   // px::hip
