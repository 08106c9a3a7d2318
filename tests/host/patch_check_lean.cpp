// Compile check of the lean binding headers under docs/reference_patch/include/hip_lean/ (first-writer
// shortcuts, the norm of a delta from its last writer, all heads in one pass, one optimiser step for all
// layers) against reference_stub.h, as patch_check.cpp checks the plain ones.  Nothing is linked or run.
#define PX_HIP_LEAN_BINDINGS
#include "reference_stub.h"

#include "hip/HipError.h"
#include "hip/Activation.h"
#include "hip_lean/ModelExtras.h"
#include "hip_lean/Layer.h"
#include "hip_lean/Model.h"
#include "hip/Adam.h"
#include "hip_lean/MaxPoolLayer.h"
#include "hip/UpsampleLayer.h"
#include "hip/RouteLayer.h"
#include "hip_lean/ShortcutLayer.h"
#include "hip/BatchNormLayer.h"
#include "hip_lean/ConvLayer.h"
#include "hip_lean/YoloLayer.h"

namespace px {
template class Model<Device::HIP>;
template class MaxPoolLayer<Device::HIP>;
template class UpsampleLayer<Device::HIP>;
template class RouteLayer<Device::HIP>;
template class ShortcutLayer<Device::HIP>;
template class BatchNormLayer<Device::HIP>;
template class ConvLayer<Device::HIP>;
template class YoloLayer<Device::HIP>;
template class Adam<Device::HIP>;
}   // px
