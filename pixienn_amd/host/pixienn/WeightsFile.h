// The weights file of a model, in the reference's layout (include/Model.h:1272-1295 reader,
// 1973-1985 writer):
//
//   int32 major, int32 minor, int32 revision      (0.1.0 for files this engine writes first)
//   seen: the images trained on -- 64 bits when major*10 + minor >= 2 (and both < 1000), 32 bits
//         otherwise (the Darknet convention the reader follows)
//   then, for every layer in network order, what its saveWeights() writes: a conv layer writes
//   biases [, scales, rolling mean, rolling variance when batch-normalised], weights; a batch-norm
//   layer biases, scales, rolling mean, rolling variance; every other layer nothing.
//
// The reader insists that the layers consume the file exactly.  The reference's writer always
// stores `seen` in 32 bits, which its own reader cannot read back once the version is 0.2 or
// later; here the width follows the version on both sides, so every file written can be read.
#pragma once

#include <cstdint>
#include <istream>
#include <ostream>
#include <string>
#include <vector>

#include "Layer.h"

namespace px::hip {

struct WeightsHeader
{
    std::int32_t major = 0, minor = 1, revision = 0;
    std::uint64_t seen = 0;

    bool wideSeen() const noexcept { return major * 10 + minor >= 2 && major < 1000 && minor < 1000; }
};

inline WeightsHeader readWeightsHeader(std::istream& is)
{
    WeightsHeader h;
    is.read(reinterpret_cast<char*>(&h.major), sizeof(h.major));
    is.read(reinterpret_cast<char*>(&h.minor), sizeof(h.minor));
    is.read(reinterpret_cast<char*>(&h.revision), sizeof(h.revision));
    if (h.wideSeen()) {
        is.read(reinterpret_cast<char*>(&h.seen), sizeof(h.seen));
    } else {
        std::uint32_t seen = 0;
        is.read(reinterpret_cast<char*>(&seen), sizeof(seen));
        h.seen = seen;
    }
    PX_CHECK(is.good(), "Could not read the weights file header");
    return h;
}

inline void writeWeightsHeader(std::ostream& os, const WeightsHeader& h)
{
    os.write(reinterpret_cast<const char*>(&h.major), sizeof(h.major));
    os.write(reinterpret_cast<const char*>(&h.minor), sizeof(h.minor));
    os.write(reinterpret_cast<const char*>(&h.revision), sizeof(h.revision));
    if (h.wideSeen()) {
        os.write(reinterpret_cast<const char*>(&h.seen), sizeof(h.seen));
    } else {
        const auto seen = static_cast<std::uint32_t>(h.seen);
        os.write(reinterpret_cast<const char*>(&seen), sizeof(seen));
    }
    PX_CHECK(os.good(), "Could not write the weights file header");
}

// Reads a whole weights file into the layers; throws unless the layers consume it exactly.
inline WeightsHeader loadWeightsFile(std::istream& is, const std::vector<Layer::Ptr>& layers)
{
    is.seekg(0, std::istream::end);
    const std::streamoff length = is.tellg();
    is.seekg(0, std::istream::beg);
    const WeightsHeader h = readWeightsHeader(is);
    std::streamoff pos = is.tellg();
    for (const auto& layer: layers) pos += layer->loadWeights(is);
    PX_CHECK(pos == length, "Did not fully read weights file; read " + std::to_string(pos) + " bytes, expected to read " +
                            std::to_string(length) + " bytes.");
    return h;
}

inline void saveWeightsFile(std::ostream& os, const WeightsHeader& h, const std::vector<Layer::Ptr>& layers)
{
    writeWeightsHeader(os, h);
    for (const auto& layer: layers) layer->saveWeights(os);
    PX_CHECK(os.good(), "Could not write the weights file");
}

}   // px::hip
