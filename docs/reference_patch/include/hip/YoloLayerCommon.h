// include/hip/YoloLayerCommon.h -- the parts of the YOLO layer's HIP binding that do not depend on when the
// training forward runs: the layer's device-side extras, setup(), the ground-truth upload, the collection of
// cost and statistics, and the detections (replaces include/cuda/YoloLayer.h:25-69, 132-188).  YoloLayer<D>
// gains two private helpers, uploadTruths() and collectCost(), declared beside setup().
#pragma once

#include <algorithm>

#include "HipError.h"

namespace px {

template<>
class YoloExtras<Device::HIP>
{
protected:
    static constexpr int kStats = 12;
    PxHipVector statsGpu_, costGpu_, truthsGpu_;
    PxHipVectorT<int> truthCountsGpu_, detectionCount_;
    PxHipVector detectionRecords_;           // capacity * 8 words
    PxCpuVector hostTruths_;
    PxCpuVectorT<int> hostTruthCounts_;
    unsigned truthCapacity_ = 0;
    int detectionCapacity_ = 0;
};

template<>
inline void YoloLayer<Device::HIP>::setup()
{
    statsGpu_ = PxHipVector(kStats);
    costGpu_ = PxHipVector(1);
    hostTruthCounts_ = PxCpuVectorT<int>(this->batch(), 0);
    truthCountsGpu_ = PxHipVectorT<int>(this->batch());
    detectionCapacity_ = 1 << 16;
    detectionRecords_ = PxHipVector(static_cast<std::size_t>(detectionCapacity_) * sizeof(pxh_detection) / sizeof(float));
    detectionCount_ = PxHipVectorT<int>(1);
}

// The ground truth of the batch as the library takes it: [batch][capacity][5] floats and a count per image.
template<>
inline void YoloLayer<Device::HIP>::uploadTruths()
{
    auto maxTruth = 1u;
    for (auto b = 0; b < this->batch(); ++b)
        maxTruth = std::max(maxTruth, static_cast<unsigned>(this->groundTruth(b).size()));
    if (maxTruth > truthCapacity_) {
        truthCapacity_ = maxTruth;
        hostTruths_ = PxCpuVector(this->batch() * truthCapacity_ * 5, 0.0f);
        truthsGpu_ = PxHipVector(hostTruths_.size());
    }
    std::fill(hostTruths_.begin(), hostTruths_.end(), 0.0f);
    for (auto b = 0; b < this->batch(); ++b) {
        const auto& truths = this->groundTruth(b);
        hostTruthCounts_[b] = static_cast<int>(truths.size());
        for (auto t = 0u; t < truths.size(); ++t) {
            const auto at = (b * truthCapacity_ + t) * 5;
            hostTruths_[at] = truths[t].box.x();
            hostTruths_[at + 1] = truths[t].box.y();
            hostTruths_[at + 2] = truths[t].box.w();
            hostTruths_[at + 3] = truths[t].box.h();
            hostTruths_[at + 4] = static_cast<float>(truths[t].classId);
        }
    }
    truthsGpu_.copy(hostTruths_);
    truthCountsGpu_.copy(hostTruthCounts_);
}

// The cost and, when training, the statistics of the last training forward (include/cuda/YoloLayer.h:132-148:
// a validating pass has ground truth and a cost but must not add to the training statistics or log).
template<>
inline void YoloLayer<Device::HIP>::collectCost()
{
    const auto cost = costGpu_.asVector();          // waits for the launch; defer to the logging step if it matters
    this->cost_ = cost[0] / std::max(1, this->batch());
    if (!this->training()) return;
    const auto stats = statsGpu_.asVector();
    avgIoU_ += stats[0]; recall_ += stats[1]; recall75_ += stats[2];
    avgCat_ += stats[3]; avgObj_ += stats[4]; avgAnyObj_ += stats[5];
    count_ += static_cast<int>(stats[6]); classCount_ += static_cast<int>(stats[7]);
    boxCost_ = stats[8];
    objectCost_ = stats[9];
    noObjectCost_ = stats[10];
    classCost_ = stats[11];
    if (count_ > 0 && this->model().seen() % logInterval_ == 0) {
        writeStats();
        resetStats();
    }
}

// image size 0 x 0: boxes relative to the network input
template<>
inline void YoloLayer<Device::HIP>::addDetects(Detections& detects, int width, int height, float threshold)
{
    auto* records = reinterpret_cast<pxh_detection*>(detectionRecords_.data());
    detectionCount_.fill(0);
    PX_HIP_CHECK(pxh_yolo_detections(this->output_.data(), this->batch(), mask_.data(), numMasks_, anchors_.data(),
                                     numAnchors_, this->classes(), this->width(), this->height(), this->model().width(),
                                     this->model().height(), width, height, threshold, records, detectionCapacity_,
                                     detectionCount_.data(), nullptr));
    // the count first (4 bytes), then the records that were found and no more: a trained network leaves a few
    // dozen, the buffer holds 65536
    const int found = std::min(detectionCount_.asVector()[0], detectionCapacity_);
    std::vector<pxh_detection> host(static_cast<std::size_t>(found));
    if (found > 0) detectionRecords_.copyToHost(reinterpret_cast<float*>(host.data()), host.size() * sizeof(pxh_detection) / sizeof(float));
    // the order in which the reference's loops emit them (image, cell, mask, class)
    std::sort(host.begin(), host.end(), [](const pxh_detection& a, const pxh_detection& b) { return a.order < b.order; });
    for (const auto& r: host)
        detects.emplace_back(cv::Rect2f{ r.x, r.y, r.w, r.h }, r.batch, r.class_index, r.prob);
}

template<>
inline void YoloLayer<Device::HIP>::addDetects(Detections& detects, float threshold)
{
    addDetects(detects, 0, 0, threshold);
}

}   // px
