// include/hip/Activation.h -- activations on the device (replaces the CUDA part of include/Activation.h:250-262
// and the kernels of include/Activation.cuh).  The layer bindings pass the activation's id to the fused
// kernels, so the interface gains type(); apply() and gradient() stay for callers outside the layers.
#pragma once

#include "HipError.h"

namespace px {

template<>
class IActivation<Device::HIP>
{
public:
    using V = PxHipVector;
    using T = float;

    virtual ~IActivation() = default;
    virtual ActivationType type() const noexcept = 0;      // LEAKY .. TANH == PXH_LEAKY .. PXH_TANH

    void apply(T* begin, T* end) const
    {
        PX_HIP_CHECK(pxh_activate(type(), begin, static_cast<std::size_t>(end - begin), nullptr));
    }

    void apply(V& container) const { apply(container.data(), container.data() + container.size()); }

    // delta *= f'(x), x = the values BEFORE the activation
    void gradient(const V& container, V& delta) const
    {
        PX_HIP_CHECK(pxh_gradient(type(), container.data(), delta.size(), delta.data(), nullptr));
    }
};

static_assert(int(LEAKY) == int(PXH_LEAKY) && int(LINEAR) == int(PXH_LINEAR) && int(LOGGY) == int(PXH_LOGGY) &&
              int(LOGISTIC) == int(PXH_LOGISTIC) && int(MISH) == int(PXH_MISH) && int(RELU) == int(PXH_RELU) &&
              int(SOFTPLUS) == int(PXH_SOFTPLUS) && int(SWISH) == int(PXH_SWISH) && int(TANH) == int(PXH_TANH),
              "include/ActivationTypes.h and pixienn_hip.h number the activations alike");

}   // px
