// include/hip_lean/MaxPoolLayer.h -- include/hip/MaxPoolLayer.h whose forward has nothing left to do when the
// pool RIDES on the epilogue of the convolution in front of it (DeviceExtras<HIP>::carryPool, at inference, for the
// 2 x 2 window at stride 2 over planes of even size: five of the six pools of YOLOv3-tiny): that convolution writes
// this layer's output in its own pass (pxh_bn_folded_act_maxpool_forward, hip_lean/ConvLayer.h).
#pragma once

#include "Layer.h"

namespace px {

template<>
class MPExtras<Device::HIP>
{
protected:
    PxHipVectorT<int> indexes_;
};

template<>
inline void MaxPoolLayer<Device::HIP>::setup()
{
    indexes_ = PxHipVectorT<int>(this->batch() * this->outputs(), -1);
}

template<>
inline void MaxPoolLayer<Device::HIP>::forward(const V& input)
{
    Layer<Device::HIP>::forward(input);
    if (this->model().rides(this)) return;
    PX_HIP_CHECK(pxh_maxpool_forward(input.data(), this->output_.data(), indexes_.data(), this->batch(), this->channels(),
                                     this->height(), this->width(), this->outHeight(), this->outWidth(), kernel_, stride_,
                                     padding_, nullptr));
}

template<>
inline void MaxPoolLayer<Device::HIP>::backward(const V& input, V* grad)
{
    Layer<Device::HIP>::backward(input, grad);
    if (grad == nullptr) return;
    PX_HIP_CHECK(pxh_maxpool_backward(this->delta_.data(), indexes_.data(), grad->data(), this->batch(), this->channels(),
                                      this->height(), this->width(), this->outHeight(), this->outWidth(), kernel_,
                                      stride_, padding_, nullptr));
}

}   // px
