// include/hip_lean/Model.h -- Model<Device::HIP>::update (replaces the loop of include/Model.h:1784-1792).
#pragma once

#include "ModelExtras.h"

namespace px {

// Model<D>::update with the parameter tensors of all layers stepped together.  The layers' own update() bodies
// (include/hip/ConvLayer.h, BatchNormLayer.h) are not called: what they do per tensor -- the two hooks on each
// update buffer, then Adam or SGD -- is what the tables do for all tensors.  The hooks' second pass over every
// layer's delta_ (Layer<D>::update, include/Layer.h:400-411) is dropped: backward has consumed the deltas by
// then and the next forward clears them, so nothing reads the result.
template<>
inline void Model<Device::HIP>::update()
{
    ++optimizerStep_;
    updateLR();
    this->updateAll(gradRescaling(), gradThreshold(), gradClipping(), gradClipValue(), adamEnabled(), updateBatch(),
                    updateCount(), learningRate(), momentum(), adamBeta1(), adamBeta2(), adamEpsilon(), decay());
}

}   // px
