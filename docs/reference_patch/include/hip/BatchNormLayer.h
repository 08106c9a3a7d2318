// include/hip/BatchNormLayer.h -- replaces include/cuda/BatchNormLayer.h:59-184 (cuDNN batch normalisation,
// cuBLAS momentum steps).  Numerics follow the CPU layer (include/BatchNormLayer.h:100-181, src/CpuUtil.cpp),
// not cuDNN: 1/(sqrt(var) + 1e-5) forward, 1/sqrt(var + 1e-5) backward.
#pragma once

#include "Layer.h"

namespace px {

template<>
class BNExtras<Device::HIP>
{
};

template<>
inline void BatchNormLayer<Device::HIP>::setup()
{
}

template<>
inline void BatchNormLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    const int spatial = this->outHeight() * this->outWidth();
    if (training()) {
        // the input is kept as it is (backward is handed it again), so no x_ copy and no xNorm_
        PX_HIP_CHECK(pxh_bn_train_act_forward(input.data(), output_.data(), nullptr, nullptr, nullptr, mean_.data(),
                                              var_.data(), rollingMean_.data(), rollingVar_.data(), scales_.data(),
                                              biases_.data(), this->batch(), this->outChannels(), spatial, PXH_LINEAR,
                                              nullptr, 0, nullptr));
    } else {
        PX_HIP_CHECK(pxh_bn_infer_act_forward(input.data(), output_.data(), nullptr, rollingMean_.data(),
                                              rollingVar_.data(), scales_.data(), biases_.data(), this->batch(),
                                              this->outChannels(), spatial, PXH_LINEAR, nullptr, 0, nullptr));
    }
}

template<>
inline void BatchNormLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    // in place on delta_; accumulates into the two update buffers
    PX_HIP_CHECK(pxh_bn_act_backward(delta_.data(), input.data(), nullptr, mean_.data(), var_.data(), scales_.data(),
                                     biases_.data(), scaleUpdates_.data(), biasUpdates_.data(), nullptr, nullptr,
                                     this->batch(), this->outChannels(), this->outHeight() * this->outWidth(), PXH_LINEAR,
                                     nullptr, 0, nullptr));
    if (grad != nullptr) PX_HIP_CHECK(pxh_axpy(delta_.size(), 1.0f, delta_.data(), grad->data(), nullptr));
}

template<>
inline void BatchNormLayer<Device::HIP>::update()
{
    const auto& net = this->model();
    Layer<Device::HIP>::update();
    // plain momentum steps, no weight decay (include/BatchNormLayer.h:166-181)
    PX_HIP_CHECK(pxh_sgd_update(biases_.size(), biases_.data(), biasUpdates_.data(), net.updateBatch(), net.learningRate(),
                                net.momentum(), 0.0f, 0, nullptr));
    PX_HIP_CHECK(pxh_sgd_update(scales_.size(), scales_.data(), scaleUpdates_.data(), net.updateBatch(),
                                net.learningRate(), net.momentum(), 0.0f, 0, nullptr));
}

template<>
inline void BatchNormLayer<Device::HIP>::scaleGradients()
{
    Layer<Device::HIP>::scaleGradients();
    this->scaleTensor(biasUpdates_);
    this->scaleTensor(scaleUpdates_);
}

template<>
inline void BatchNormLayer<Device::HIP>::clipGradients()
{
    Layer<Device::HIP>::clipGradients();
    PX_HIP_CHECK(pxh_constrain(static_cast<int>(biasUpdates_.size()), this->gradientClipValue_, biasUpdates_.data(), nullptr));
    PX_HIP_CHECK(pxh_constrain(static_cast<int>(scaleUpdates_.size()), this->gradientClipValue_, scaleUpdates_.data(), nullptr));
}

}   // px
