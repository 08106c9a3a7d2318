// include/hip_lean/ConvLayer.h -- ConvLayer<Device::HIP> with three things the plain bodies cannot know:
//   * setup() hands the layer's parameter tensors to the model, so that Model<HIP>::update (Model.h here) steps
//     the tensors of all layers together: the layer's own update() is then never called;
//   * a ShortcutLayer that RIDES on this layer (DeviceExtras<HIP>::carry, for a residual block: nothing but the
//     shortcut reads this layer's output, the shortcut is linear over tensors of one shape): forward writes the
//     shortcut's output in the epilogue's own pass (pxh_bn_train_act_shortcut_forward: the shortcut's 12 bytes
//     per element become 4 more read here, this layer's own output_ is never formed), and backward works on the
//     shortcut's delta as this layer's own (alpha = 1: the two hold the same values; the shortcut's helpers have
//     been over it, and this layer's repeat without changing a value, as they would on the copy).
//   * a MaxPoolLayer that rides on this layer at inference (DeviceExtras<HIP>::carryPool): the epilogue writes the
//     pool's output in its own pass (pxh_bn_folded_act_maxpool_forward), and this layer's own only when a route
//     reads it as well.
// Everything else as in include/hip/ConvLayer.h.
#pragma once

#include "Layer.h"
#include "../hip/ConvLayerCommon.h"

namespace px {

template<>
inline void ConvLayer<Device::HIP>::setup()
{
    // ... the engine's own setup of the layer's tensors (include/ConvLayer.h:129-190), then:
    const auto& net = this->model();
    net.registerParameters(weights_, weightUpdates_, m_, v_, true);
    net.registerParameters(biases_, biasUpdates_, bias_m_, bias_v_, false);
    if (scales_.size()) net.registerParameters(scales_, scaleUpdates_, scale_m_, scale_v_, false);
}

template<>
inline void ConvLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    const int spatial = this->outHeight() * this->outWidth();
    const int act = activation_->type();
    const auto* rider = batchNorm_ ? this->model().riderOf(this) : nullptr;
    if (batchNorm_ && training()) {
        convolveForward(input, weights_, x_);
        if (rider)
            PX_HIP_CHECK(pxh_bn_train_act_shortcut_forward(x_.data(), rider->output->data(), nullptr, nullptr, nullptr,
                                                           mean_.data(), var_.data(), rollingMean_.data(),
                                                           rollingVar_.data(), scales_.data(), biases_.data(),
                                                           rider->from->data(), rider->alpha, rider->beta, this->batch(),
                                                           filters_, spatial, act, nullptr, 0, nullptr));
        else
            PX_HIP_CHECK(pxh_bn_train_act_forward(x_.data(), this->output_.data(), nullptr, nullptr, nullptr, mean_.data(),
                                                  var_.data(), rollingMean_.data(), rollingVar_.data(), scales_.data(),
                                                  biases_.data(), this->batch(), filters_, spatial, act, nullptr, 0,
                                                  nullptr));
        foldedReady_ = false;
        return;
    }
    convolveForward(input, weights_, this->output_);
    if (batchNorm_) {
        if (!foldedReady_) {
            if (folded_.empty()) folded_ = V(pxh_bn_folded_bytes(filters_) / sizeof(float));
            PX_HIP_CHECK(pxh_bn_fold(rollingMean_.data(), rollingVar_.data(), scales_.data(), biases_.data(), filters_,
                                     folded_.data(), nullptr));
            foldedReady_ = true;
        }
        const auto* pool = this->model().poolOf(this);
        if (rider)
            PX_HIP_CHECK(pxh_bn_folded_act_shortcut_forward(this->output_.data(), rider->output->data(), nullptr,
                                                            folded_.data(), rider->from->data(), rider->alpha,
                                                            rider->beta, this->batch(), filters_, spatial, act, nullptr));
        else if (pool)
            // in place on the GEMM result when the layer's output is kept, else that tensor is only read
            PX_HIP_CHECK(pxh_bn_folded_act_maxpool_forward(this->output_.data(),
                                                           pool->keepOutput ? this->output_.data() : nullptr,
                                                           pool->pooled->data(), folded_.data(), this->batch(), filters_,
                                                           this->outHeight(), this->outWidth(), act, nullptr));
        else
            PX_HIP_CHECK(pxh_bn_folded_act_forward(this->output_.data(), this->output_.data(), nullptr, folded_.data(),
                                                   this->batch(), filters_, spatial, act, nullptr));
    } else {
        float* pre = training() && act != LINEAR ? this->preActivation_.data() : nullptr;
        PX_HIP_CHECK(pxh_bias_act_forward(this->output_.data(), this->output_.data(), pre, biases_.data(), this->batch(),
                                          filters_, spatial, act, nullptr));
    }
}

template<>
inline void ConvLayer<Device::HIP>::backward(const V& input, V* grad)
{
    const float threshold = this->gradientRescaling_ ? this->gradientThreshold_ : 0.0f;
    const float clip = this->gradientClipping_ ? this->gradientClipValue_ : 0.0f;
    const int spatial = this->outHeight() * this->outWidth();
    const int act = activation_->type();
    const auto* rider = batchNorm_ ? this->model().riderOf(this) : nullptr;
    V& delta = rider ? *rider->delta : this->delta_;
    if (batchNorm_) {
        PX_HIP_CHECK(pxh_bn_act_backward_clipped(delta.data(), x_.data(), nullptr, mean_.data(), var_.data(),
                                                 scales_.data(), biases_.data(), scaleUpdates_.data(),
                                                 biasUpdates_.data(), nullptr, nullptr, this->batch(), filters_, spatial,
                                                 act, threshold, clip, nullptr, nullptr, 0, nullptr));
    } else {
        const float* pre = act != LINEAR ? this->preActivation_.data() : nullptr;
        PX_HIP_CHECK(pxh_bias_act_backward_clipped(delta.data(), pre, biasUpdates_.data(), this->batch(), filters_,
                                                   spatial, act, threshold, clip, nullptr, nullptr, 0, nullptr));
    }
    convolveBackward(input, weights_, delta, weightUpdates_, grad);
}

}   // px
