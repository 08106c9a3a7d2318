// include/hip_lean/ShortcutLayer.h -- include/hip/ShortcutLayer.h with the backward of a same-shape shortcut as
// the FIRST writer of the two deltas it reaches (the layer in front of it and its `from` layer: in a residual
// block nothing else has written them when the shortcut's backward runs) and as the LAST writer of the first
// of them: it overwrites instead of adding into cleared tensors, and leaves that delta's norm and peak behind.
// Whoever builds the graph marks the two deltas (DeviceExtras<HIP>::markOverwritten) when that holds -- or lets
// the shortcut ride on the convolution in front of it (DeviceExtras<HIP>::carry), which then writes this layer's
// output and takes this layer's delta: forward has nothing left to do here, backward only the `from` layer's share.
#pragma once

#include "Layer.h"
#include "../hip/Activation.h"

namespace px {

template<>
inline void ShortcutLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    if (this->model().rides(this)) return;      // the convolution in front has written output_ (hip_lean/ConvLayer.h)
    const bool sameShape = from_->outWidth() == this->outWidth() && from_->outHeight() == this->outHeight() &&
                           from_->outChannels() == this->outChannels();
    float* pre = preActivation_.empty() ? nullptr : preActivation_.data();
    if (sameShape) {
        PX_HIP_CHECK(pxh_shortcut_forward(input.data(), from_->output().data(), this->output_.data(), pre,
                                          this->output_.size(), alpha_, beta_, activation_->type(), nullptr));
        return;
    }
    this->output_.copy(input);
    PX_HIP_CHECK(pxh_shortcut(this->batch(), this->width(), this->height(), this->channels(), from_->output().data(),
                              this->outWidth(), this->outHeight(), this->outChannels(), alpha_, beta_,
                              this->output_.data(), nullptr));
    if (pre) preActivation_.copy(this->output_);
    activation_->apply(this->output_);
}

template<>
inline void ShortcutLayer<Device::HIP>::backward(const V& input, V* grad)
{
    const auto& net = this->model();
    const bool sameShape = from_->outWidth() == this->outWidth() && from_->outHeight() == this->outHeight() &&
                           from_->outChannels() == this->outChannels();
    const float* pre = preActivation_.empty() ? nullptr : preActivation_.data();
    // A riding shortcut that is the first to write its `from` layer's delta: the rescale + clip of delta_ that opens
    // every layer's backward and the shortcut's own backward as ONE call, which reads delta_ once when nothing has
    // to change (pxh_shortcut_backward_clipped: the values of the two calls to the bit).
    const float threshold = this->gradientRescaling_ ? this->gradientThreshold_ : 0.0f;
    const float clip = this->gradientClipping_ ? this->gradientClipValue_ : 0.0f;
    if (net.rides(this) && net.overwritten(from_->delta().data()) && (threshold > 0.0f || clip > 0.0f) &&
        !net.hasNormGroups(this->delta_.data())) {
        PX_HIP_CHECK(pxh_shortcut_backward_clipped(this->delta_.data(), nullptr, from_->delta().data(), nullptr,
                                                   this->delta_.size(), alpha_, beta_, activation_->type(), 1, threshold,
                                                   clip, nullptr, nullptr, 0, nullptr));
        return;
    }
    Layer<Device::HIP>::backward(input, grad);
    if (net.rides(this)) {
        // the `from` layer's share only: the convolution in front works on delta_ itself
        if (net.overwritten(from_->delta().data()))
            PX_HIP_CHECK(pxh_shortcut_backward_first(this->delta_.data(), nullptr, from_->delta().data(), nullptr,
                                                     this->delta_.size(), alpha_, beta_, activation_->type(), nullptr));
        else
            PX_HIP_CHECK(pxh_shortcut_backward(this->delta_.data(), nullptr, from_->delta().data(), nullptr,
                                               this->delta_.size(), alpha_, beta_, activation_->type(), nullptr));
        return;
    }
    if (sameShape && grad != nullptr) {
        const bool first = net.overwritten(grad->data()) && net.overwritten(from_->delta().data());
        PxHipVector& groups = net.normGroupsFor(this, grad->size());
        PX_HIP_CHECK(pxh_shortcut_backward_norm(this->delta_.data(), pre, from_->delta().data(), grad->data(),
                                                this->delta_.size(), alpha_, beta_, activation_->type(), first ? 1 : 0,
                                                groups.data(), nullptr));
        net.noteNormGroups(grad->data(), groups.data());
        return;
    }
    if (sameShape) {
        PX_HIP_CHECK(pxh_shortcut_backward(this->delta_.data(), pre, from_->delta().data(), nullptr, this->delta_.size(),
                                           alpha_, beta_, activation_->type(), nullptr));
        return;
    }
    if (activation_->type() != LINEAR) activation_->gradient(preActivation_, this->delta_);
    PX_HIP_CHECK(pxh_shortcut(this->batch(), this->outWidth(), this->outHeight(), this->outChannels(),
                              this->delta_.data(), this->width(), this->height(), this->channels(), 1.0f, beta_,
                              from_->delta().data(), nullptr));
    if (grad != nullptr)
        PX_HIP_CHECK(pxh_axpy(this->delta_.size(), alpha_, this->delta_.data(), grad->data(), nullptr));
}

}   // px
