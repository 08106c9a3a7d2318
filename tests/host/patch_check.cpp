// Compile check of the binding headers under docs/reference_patch/include/hip/ against
// reference_stub.h: every method body must name only members the engine's classes have and call the
// library with arguments of the declared types.  Instantiating the layer classes makes the compiler
// check the specialisations against the class definitions; nothing here is linked or run.
#include "reference_stub.h"

#include "hip/HipError.h"
#include "hip/Activation.h"
#include "hip/Layer.h"
#include "hip/Adam.h"
#include "hip/MaxPoolLayer.h"
#include "hip/UpsampleLayer.h"
#include "hip/RouteLayer.h"
#include "hip/ShortcutLayer.h"
#include "hip/BatchNormLayer.h"
#include "hip/ConvLayerCommon.h"
#include "hip/ConvLayer.h"
#include "hip/YoloLayerCommon.h"
#include "hip/YoloLayer.h"

namespace px {
template class MaxPoolLayer<Device::HIP>;
template class UpsampleLayer<Device::HIP>;
template class RouteLayer<Device::HIP>;
template class ShortcutLayer<Device::HIP>;
template class BatchNormLayer<Device::HIP>;
template class ConvLayer<Device::HIP>;
template class YoloLayer<Device::HIP>;
template class Adam<Device::HIP>;
}   // px
