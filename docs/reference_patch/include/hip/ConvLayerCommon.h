// include/hip/ConvLayerCommon.h -- what the plain and the lean ConvLayer bodies share.  Together with
// ConvLayer.h: everything of include/cuda/ConvLayer.h:266-434 except the convolution itself:
// the batch-norm / bias / activation epilogue after the forward GEMM, its mirror image before the backward
// GEMMs, the optimiser step and the gradient hooks.  The three convolution calls (cudnnConvolutionForward,
// BackwardFilter, BackwardData there; MIOpen or a GEMM of the engine's choice here) are the two hooks of
// CVExtras<Device::HIP> and are not part of this library.
#pragma once

#include "Activation.h"
#include "Adam.h"
#include "Layer.h"

namespace px {

template<>
class CVExtras<Device::HIP>
{
protected:
    using V = PxHipVector;

    // y = conv(input, weights); the engine's own
    void convolveForward(const V& input, const V& weights, V& y);
    // weightUpdates += d(conv)/d(weights); if grad: *grad += d(conv)/d(input); the engine's own
    void convolveBackward(const V& input, const V& weights, const V& delta, V& weightUpdates, V* grad);

    V m_, v_, bias_m_, bias_v_, scale_m_, scale_v_;     // Adam moments
    V folded_;                                          // per-channel constants of the inference epilogue
    bool foldedReady_ = false;
};

template<>
inline void ConvLayer<Device::HIP>::update()
{
    const auto& net = this->model();
    Layer<Device::HIP>::update();
    foldedReady_ = false;
    if (net.adamEnabled()) {
        Adam<Device::HIP> adam(net.updateBatch(), net.updateCount(), net.learningRate(), net.adamBeta1(),
                               net.adamBeta2(), net.adamEpsilon(), net.decay());
        adam.update(weights_, weightUpdates_, m_, v_, true);
        adam.update(biases_, biasUpdates_, bias_m_, bias_v_, false);
        if (scales_.size()) adam.update(scales_, scaleUpdates_, scale_m_, scale_v_, false);
        return;
    }
    // SGD with momentum: one launch per tensor for the three cuBLAS calls each (decay on the weights only)
    PX_HIP_CHECK(pxh_sgd_update(weights_.size(), weights_.data(), weightUpdates_.data(), net.updateBatch(),
                                net.learningRate(), net.momentum(), net.decay(), 1, nullptr));
    PX_HIP_CHECK(pxh_sgd_update(biases_.size(), biases_.data(), biasUpdates_.data(), net.updateBatch(), net.learningRate(),
                                net.momentum(), net.decay(), 0, nullptr));
    if (scales_.size())
        PX_HIP_CHECK(pxh_sgd_update(scales_.size(), scales_.data(), scaleUpdates_.data(), net.updateBatch(),
                                    net.learningRate(), net.momentum(), net.decay(), 0, nullptr));
}

template<>
inline void ConvLayer<Device::HIP>::scaleGradients()
{
    Layer<Device::HIP>::scaleGradients();
    this->scaleTensor(weightUpdates_);
    this->scaleTensor(biasUpdates_);
    if (scaleUpdates_.size()) this->scaleTensor(scaleUpdates_);
}

template<>
inline void ConvLayer<Device::HIP>::clipGradients()
{
    Layer<Device::HIP>::clipGradients();
    PX_HIP_CHECK(pxh_constrain(static_cast<int>(weightUpdates_.size()), this->gradientClipValue_, weightUpdates_.data(),
                               nullptr));
    PX_HIP_CHECK(pxh_constrain(static_cast<int>(biasUpdates_.size()), this->gradientClipValue_, biasUpdates_.data(), nullptr));
    if (scaleUpdates_.size())
        PX_HIP_CHECK(pxh_constrain(static_cast<int>(scaleUpdates_.size()), this->gradientClipValue_, scaleUpdates_.data(),
                                   nullptr));
}

}   // px
