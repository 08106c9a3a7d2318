// include/hip/UpsampleLayer.h -- replaces include/cuda/UpsampleLayer.h:23-51 (upsampleGpu, same argument order).
#pragma once

#include "HipError.h"

namespace px {

template<>
class UpsampleExtras<Device::HIP>
{
};

template<>
inline void UpsampleLayer<Device::HIP>::setup()
{
}

template<>
inline void UpsampleLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    PX_HIP_CHECK(pxh_upsample(input.data(), this->width(), this->height(), this->channels(), this->batch(), stride_, 1,
                              scale_, nullptr, this->output_.data(), nullptr));
}

template<>
inline void UpsampleLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    if (grad == nullptr) return;
    PX_HIP_CHECK(pxh_upsample(nullptr, this->width(), this->height(), this->channels(), this->batch(), stride_, 0, scale_,
                              grad->data(), this->delta_.data(), nullptr));
}

}   // px
