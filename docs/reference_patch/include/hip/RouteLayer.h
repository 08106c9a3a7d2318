// include/hip/RouteLayer.h -- replaces include/cuda/RouteLayer.h:23-71: one launch per source layer
// instead of batch x layers cudaMemcpy / cublasSaxpy calls.
#pragma once

#include "HipError.h"

namespace px {

template<>
inline void RouteLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    auto offset = 0;
    for (const auto& layer: layers_) {
        PX_HIP_CHECK(pxh_route_forward(layer->output().data(), this->output_.data(), this->batch(), layer->outputs(),
                                       this->outputs(), offset, nullptr));
        offset += layer->outputs();
    }
}

template<>
inline void RouteLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    auto offset = 0;
    for (const auto& layer: layers_) {
        PX_HIP_CHECK(pxh_route_backward(this->delta_.data(), layer->delta().data(), this->batch(), layer->outputs(),
                                        this->outputs(), offset, nullptr));
        offset += layer->outputs();
    }
}

}   // px
