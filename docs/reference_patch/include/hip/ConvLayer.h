// include/hip/ConvLayer.h -- forward and backward of ConvLayer<Device::HIP>: the batch-norm / bias / activation
// epilogue after the forward GEMM and its mirror image before the backward GEMMs (include/cuda/ConvLayer.h:266-338).
// The rest of the layer is in ConvLayerCommon.h.
#pragma once

#include "ConvLayerCommon.h"

namespace px {

template<>
inline void ConvLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    const int spatial = this->outHeight() * this->outWidth();
    const int act = activation_->type();
    if (batchNorm_ && training()) {
        // the GEMM writes x_ directly (the CUDA path copies output_ there); the pass that applies the
        // normalisation recomputes what backward needs, so neither preActivation_ nor xNorm_ is written
        convolveForward(input, weights_, x_);
        PX_HIP_CHECK(pxh_bn_train_act_forward(x_.data(), this->output_.data(), nullptr, nullptr, nullptr, mean_.data(),
                                              var_.data(), rollingMean_.data(), rollingVar_.data(), scales_.data(),
                                              biases_.data(), this->batch(), filters_, spatial, act, nullptr, 0,
                                              nullptr));
        foldedReady_ = false;
        return;
    }
    convolveForward(input, weights_, this->output_);
    if (batchNorm_) {
        // inference: fold mean, variance, scale and bias into two constants per channel once, then one
        // pass in place on the GEMM result
        if (!foldedReady_) {
            if (folded_.empty()) folded_ = V(pxh_bn_folded_bytes(filters_) / sizeof(float));
            PX_HIP_CHECK(pxh_bn_fold(rollingMean_.data(), rollingVar_.data(), scales_.data(), biases_.data(), filters_,
                                     folded_.data(), nullptr));
            foldedReady_ = true;
        }
        PX_HIP_CHECK(pxh_bn_folded_act_forward(this->output_.data(), this->output_.data(), nullptr, folded_.data(),
                                               this->batch(), filters_, spatial, act, nullptr));
    } else {
        // bias + activation; training keeps the pre-activation values for backward unless the activation
        // is linear
        float* pre = training() && act != LINEAR ? this->preActivation_.data() : nullptr;
        PX_HIP_CHECK(pxh_bias_act_forward(this->output_.data(), this->output_.data(), pre, biases_.data(), this->batch(),
                                          filters_, spatial, act, nullptr));
    }
}

template<>
inline void ConvLayer<Device::HIP>::backward(const V& input, V* grad)
{
    // Layer<D>::backward (include/Layer.h:385-397) is scaleTensor(delta_) and clipDelta(): a read of delta_
    // for its norm, a rewrite when the norm is beyond the threshold, a clamp.  The clipped entry points take
    // the two thresholds and fold all of it into the backward's own first pass over delta_, so the base
    // class's method is not called here.
    const float threshold = this->gradientRescaling_ ? this->gradientThreshold_ : 0.0f;
    const float clip = this->gradientClipping_ ? this->gradientClipValue_ : 0.0f;
    const int spatial = this->outHeight() * this->outWidth();
    const int act = activation_->type();
    if (batchNorm_) {
        // activation gradient, batch-norm backward and `delta_.copy(xNorm_)` in one call, in place on delta_
        PX_HIP_CHECK(pxh_bn_act_backward_clipped(this->delta_.data(), x_.data(), nullptr, mean_.data(), var_.data(),
                                                 scales_.data(), biases_.data(), scaleUpdates_.data(),
                                                 biasUpdates_.data(), nullptr, nullptr, this->batch(), filters_, spatial,
                                                 act, threshold, clip, nullptr, nullptr, 0, nullptr));
    } else {
        const float* pre = act != LINEAR ? this->preActivation_.data() : nullptr;
        PX_HIP_CHECK(pxh_bias_act_backward_clipped(this->delta_.data(), pre, biasUpdates_.data(), this->batch(), filters_,
                                                   spatial, act, threshold, clip, nullptr, nullptr, 0, nullptr));
    }
    convolveBackward(input, weights_, this->delta_, weightUpdates_, grad);
}

}   // px
