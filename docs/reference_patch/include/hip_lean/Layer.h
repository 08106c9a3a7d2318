// include/hip_lean/Layer.h -- include/hip/Layer.h plus the two places where the Layer base touches delta_
// around every layer (include/Layer.h:377-397): the zero-fill in forward, skipped for a delta that the first
// backward to reach it overwrites, and the rescale + clip in backward, which starts from the norm the delta's
// last writer left behind when there is one.
#pragma once

#include "ModelExtras.h"
#include "../hip/Layer.h"

namespace px {

template<>
inline void Layer<Device::HIP>::forward(const V& /*input*/)
{
    // output_ needs no fill: every kernel of the library writes each element of its output
    if (training() && !this->model().overwritten(delta_.data())) delta_.fill(0);
    cost_ = 0;
}

template<>
inline void Layer<Device::HIP>::backward(const V& /*input*/, V* /*grad*/)
{
    const float* groups = this->model().takeNormGroups(delta_.data());
    if (!gradientRescaling_ && !gradientClipping_) return;
    const float threshold = gradientRescaling_ ? gradientThreshold_ : 0.0f;
    const float clip = gradientClipping_ ? gradientClipValue_ : 0.0f;
    if (groups)
        PX_HIP_CHECK(pxh_rescale_clip_from_groups(delta_.data(), delta_.size(), threshold, clip, nullptr, groups, nullptr, 0,
                                                  nullptr));
    else
        PX_HIP_CHECK(pxh_rescale_clip(delta_.data(), delta_.size(), threshold, clip, nullptr, nullptr, 0, nullptr));
}

}   // px
