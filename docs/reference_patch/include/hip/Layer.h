// include/hip/Layer.h -- the gradient helpers of the Layer base (replaces include/cuda/Layer.h:24-56).
// Layer<D>::backward (include/Layer.h:385-397) calls scaleTensor(delta_) and clipDelta() one after the
// other; each is one call here.  pxh_rescale_clip does both in one pass over the tensor and finds the
// norm on the device (the cuBLAS form copies it to the host and waits): an engine that wants that
// replaces the two calls in Layer<D>::backward by rescaleAndClip(delta_) below.
#pragma once

#include "HipError.h"

namespace px {

template<>
inline void Layer<Device::HIP>::scaleTensor(V& tensor)
{
    PX_HIP_CHECK(pxh_rescale_clip(tensor.data(), tensor.size(), gradientThreshold_, 0.0f, nullptr, nullptr, 0, nullptr));
}

template<>
inline void Layer<Device::HIP>::scaleGradients()
{
    scaleTensor(delta_);
}

template<>
inline void Layer<Device::HIP>::clipGradients()
{
    PX_HIP_CHECK(pxh_constrain(delta_.size(), gradientClipValue_, delta_.data(), nullptr));
}

template<>
inline void Layer<Device::HIP>::clipDelta()
{
    PX_HIP_CHECK(pxh_constrain(delta_.size(), gradientClipValue_, delta_.data(), nullptr));
}

// Both helpers at once, as the layer's flags ask for them.
inline void rescaleAndClip(PxHipVector& tensor, bool rescale, float threshold, bool clip, float clipValue)
{
    if (!rescale && !clip) return;
    PX_HIP_CHECK(pxh_rescale_clip(tensor.data(), tensor.size(), rescale ? threshold : 0.0f, clip ? clipValue : 0.0f,
                                  nullptr, nullptr, 0, nullptr));
}

}   // px
