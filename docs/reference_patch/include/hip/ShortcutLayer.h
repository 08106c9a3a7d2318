// include/hip/ShortcutLayer.h -- replaces include/cuda/ShortcutLayer.h:23-54 (copy + shortcutGpu + activation;
// gradient + shortcutGpu + cublasSaxpy), following the CPU layer (include/ShortcutLayer.h:84-111), whose
// backward differentiates at the pre-activation values.  Same-shape shortcuts (every one in the shipped
// networks) are one launch each way; differing shapes keep the index-mapped blend with the reference's own
// arguments (include/ShortcutLayer.h:91-92, 105-106).
#pragma once

#include "Activation.h"

namespace px {

template<>
inline void ShortcutLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
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
    Layer<Device::HIP>::backward(input, grad);
    const bool sameShape = from_->outWidth() == this->outWidth() && from_->outHeight() == this->outHeight() &&
                           from_->outChannels() == this->outChannels();
    const float* pre = preActivation_.empty() ? nullptr : preActivation_.data();
    if (sameShape) {
        PX_HIP_CHECK(pxh_shortcut_backward(this->delta_.data(), pre, from_->delta().data(),
                                           grad ? grad->data() : nullptr, this->delta_.size(), alpha_, beta_,
                                           activation_->type(), nullptr));
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
