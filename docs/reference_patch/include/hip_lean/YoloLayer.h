// include/hip_lean/YoloLayer.h -- include/hip/YoloLayer.h with the two things a head can leave to the model:
// its training forward waits for the end of the forward pass, where all heads of the model run as one pass
// (DeviceExtras<HIP>::forwardDeferredHeads; the cost and statistics are collected after it, by collectCost()),
// and its backward, the last writer of the delta of the layer in front of it (nothing else reads that layer's
// output in the shipped networks), leaves that delta's norm and peak behind.
#pragma once

#include "Layer.h"

#include "../hip/YoloLayerCommon.h"

namespace px {

template<>
inline void YoloLayer<Device::HIP>::forward(const V& input)
{
    // the head writes every element of delta_ itself: no fill
    this->cost_ = 0;
    const auto area = this->width() * this->height();
    if (this->inferring()) {
        PX_HIP_CHECK(pxh_yolo_activate(input.data(), this->output_.data(), this->batch(), numMasks_, this->classes(), area,
                                       nullptr));
        return;
    }
    uploadTruths();
    DeviceExtras<Device::HIP>::WaitingHead w{};
    w.head = pxh_yolo_head{ input.data(), this->output_.data(), this->delta_.data(), mask_.data(), numMasks_,
                            this->width(), this->height(), ignoreThresh_, truthThresh_, coordScale_, objectScale_,
                            noObjectScale_, classScale_, statsGpu_.data(), costGpu_.data() };
    w.anchors = anchors_.data();
    w.anchorCount = numAnchors_;
    w.batch = this->batch();
    w.classes = this->classes();
    w.truths = truthsGpu_.data();
    w.truthCounts = truthCountsGpu_.data();
    w.maxTruth = static_cast<int>(truthCapacity_);
    this->model().deferHead(w);
    // Model<D>::forward calls forwardDeferredHeads() after its last layer, then collectCost() on every head
}

template<>
inline void YoloLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    if (grad == nullptr) return;
    const auto& net = this->model();
    PxHipVector& groups = net.normGroupsFor(this, grad->size());
    PX_HIP_CHECK(pxh_axpy_norm(this->delta_.size(), 1.0f, this->delta_.data(), grad->data(), groups.data(), nullptr));
    net.noteNormGroups(grad->data(), groups.data());
}

}   // px
