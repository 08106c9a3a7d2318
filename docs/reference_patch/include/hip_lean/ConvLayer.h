// include/hip_lean/ConvLayer.h -- include/hip/ConvLayer.h whose setup() also hands the layer's parameter tensors
// to the model, so that Model<HIP>::update (Model.h here) steps the tensors of all layers together: the
// layer's own update() is then never called.
#pragma once

#include "Layer.h"
#include "../hip/ConvLayer.h"

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

}   // px
