// Device tags and traits for engine code that selects its vector type and its overloads per
// device (reference: include/DeviceTraits.h:23-56, where the tags are CPU and CUDA).  The MI355X
// path adds one tag; a layer template specialised for it takes DeviceVector<float> as its V.
#pragma once

#include <type_traits>

#include "DeviceVector.h"

namespace px::hip {

enum class Device
{
    CPU,
    HIP
};

template<Device D>
struct DeviceTraits;

template<>
struct DeviceTraits<Device::HIP>
{
    using VectorType = FloatVector;
    using ValueType = VectorType::value_type;
};

template<Device D>
struct IsHipDevice : std::false_type
{
};

template<>
struct IsHipDevice<Device::HIP> : std::true_type
{
};

template<Device D, typename T = void>
using EnableIfCpu = std::enable_if_t<!IsHipDevice<D>::value, T>;

template<Device D, typename T = void>
using EnableIfHip = std::enable_if_t<IsHipDevice<D>::value, T>;

}   // px::hip
