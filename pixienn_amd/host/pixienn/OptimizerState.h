// The Adam moments' checkpoint sidecar ("<weights>.optimizer"), byte for byte the reference's
// layout (include/Model.h:1986-2000 writer, 1306-1340 reader; per layer include/cuda/ConvLayer.h:228-264):
//
//   uint32  magic       0x50584f32 ("2OXP" on disk; 0x50584f31 is the older form without `seen`)
//   uint64  seen        images the matching weights file has seen (absent in the older form)
//   uint64  step        optimizer steps taken (std::size_t in the reference)
//   then, for every layer in network order, what its saveOptimizer() writes; a conv layer writes
//   m, v (weights), bias_m, bias_v, scale_m, scale_v as raw little-endian fp32, sizes implied by
//   the layer (scale_* are empty without batch_normalize).
#pragma once

#include <cstdint>
#include <istream>
#include <ostream>

#include "Layers.h"

namespace px::hip {

struct OptimizerHeader
{
    std::uint64_t seen = 0;
    std::uint64_t step = 0;
    bool hasSeen = true;      // false for a file of the older form
};

constexpr std::uint32_t kOptimizerMagicV1 = 0x50584f31;
constexpr std::uint32_t kOptimizerMagicV2 = 0x50584f32;

inline void writeOptimizerHeader(std::ostream& os, const OptimizerHeader& h)
{
    const std::uint32_t magic = kOptimizerMagicV2;
    os.write(reinterpret_cast<const char*>(&magic), sizeof(magic));
    os.write(reinterpret_cast<const char*>(&h.seen), sizeof(h.seen));
    os.write(reinterpret_cast<const char*>(&h.step), sizeof(h.step));
    PX_CHECK(os.good(), "Could not write optimizer state header");
}

inline OptimizerHeader readOptimizerHeader(std::istream& is)
{
    std::uint32_t magic = 0;
    is.read(reinterpret_cast<char*>(&magic), sizeof(magic));
    PX_CHECK(is.good() && (magic == kOptimizerMagicV1 || magic == kOptimizerMagicV2), "Invalid optimizer state file");
    OptimizerHeader h;
    h.hasSeen = magic == kOptimizerMagicV2;
    if (h.hasSeen) is.read(reinterpret_cast<char*>(&h.seen), sizeof(h.seen));
    is.read(reinterpret_cast<char*>(&h.step), sizeof(h.step));
    PX_CHECK(is.good(), "Could not read optimizer state header");
    return h;
}

// Writes / reads the whole sidecar for a sequence of layers (layers without optimizer state
// contribute nothing, as in the reference).  On reading, moments are only taken over when the
// file belongs to the weights (`seen` matches) - the reference discards stale moments.
inline void saveOptimizerState(std::ostream& os, const OptimizerHeader& h, const std::vector<Layer::Ptr>& layers)
{
    writeOptimizerHeader(os, h);
    for (const auto& layer: layers) layer->saveOptimizer(os);
    PX_CHECK(os.good(), "Could not write optimizer state");
}

inline bool loadOptimizerState(std::istream& is, std::uint64_t weightsSeen, OptimizerHeader& h,
                               const std::vector<Layer::Ptr>& layers)
{
    h = readOptimizerHeader(is);
    if (h.hasSeen && h.seen != weightsSeen) return false;
    for (const auto& layer: layers) layer->loadOptimizer(is);
    return true;
}

}   // px::hip
