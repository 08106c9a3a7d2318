// include/hip/YoloLayer.h -- replaces include/cuda/YoloLayer.h:70-166.  Training forward is one call:
// decode, target assignment (the host-side YoloTargetBuilder of the CUDA path), deltas, statistics and
// cost, from the uploaded ground truth alone; nothing is filled beforehand and nothing comes back until
// the loss is read.  Detections are thresholded on the device: only the records cross to the host.
#pragma once

#include "YoloLayerCommon.h"

namespace px {

template<>
inline void YoloLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    const auto area = this->width() * this->height();
    if (this->inferring()) {
        PX_HIP_CHECK(pxh_yolo_activate(input.data(), this->output_.data(), this->batch(), numMasks_, this->classes(), area,
                                       nullptr));
        return;
    }

    uploadTruths();

    PX_HIP_CHECK(pxh_yolo_forward_train(input.data(), this->output_.data(), this->delta_.data(), truthsGpu_.data(),
                                        truthCountsGpu_.data(), static_cast<int>(truthCapacity_), mask_.data(),
                                        anchors_.data(), statsGpu_.data(), costGpu_.data(), this->batch(), numMasks_,
                                        numAnchors_, this->classes(), this->width(), this->height(),
                                        this->model().width(), this->model().height(), ignoreThresh_, truthThresh_,
                                        coordScale_, objectScale_, noObjectScale_, classScale_, nullptr, 0, nullptr));

    collectCost();
}

template<>
inline void YoloLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    if (grad == nullptr) return;
    PX_HIP_CHECK(pxh_axpy(this->delta_.size(), 1.0f, this->delta_.data(), grad->data(), nullptr));
}

}   // px
