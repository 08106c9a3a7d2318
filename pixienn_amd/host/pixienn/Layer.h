// Layer interface of the MI355X kernels: the forward / backward / update / output / delta surface
// of the engine's layers (reference: include/Layer.h:43-62) over the C ABI in pixienn_hip.h.
//
// What differs from the reference, on purpose:
//   - properties come from a small key -> value map instead of a YAML node, with the reference's
//     property names and defaults;
//   - the model a layer belongs to is reduced to a Context: stream, training flag, network input
//     size, class count, ground truth of the current batch and the optimiser settings;
//   - Layer::forward does not zero-fill output_: every kernel here writes each output element.
//     delta_ is still cleared when training, because backward passes accumulate into it.
#pragma once

#include <algorithm>
#include <cmath>
#include <istream>
#include <map>
#include <ostream>
#include <memory>
#include <string>
#include <variant>
#include <unordered_map>
#include <vector>

#include "DeviceVector.h"

namespace px::hip {

// ---------------------------------------------------------------- properties
class Properties
{
public:
    using Value = std::variant<int, float, bool, std::string, std::vector<int>>;

    Properties() = default;
    Properties(std::initializer_list<std::pair<const std::string, Value>> init) : values_(init) {}

    Properties& set(const std::string& name, Value value)
    {
        values_[name] = std::move(value);
        return *this;
    }

    bool has(const std::string& name) const { return values_.count(name) != 0; }

    // Required property: throws when absent (reference: Layer<D>::property, include/Layer.h:240-250).
    template<typename T>
    T get(const std::string& name) const
    {
        auto it = values_.find(name);
        PX_CHECK(it != values_.end(), "Layer has no property named \"" + name + "\".");
        return convert<T>(it->second, name);
    }

    template<typename T>
    T get(const std::string& name, const T& def) const
    {
        auto it = values_.find(name);
        return it == values_.end() ? def : convert<T>(it->second, name);
    }

private:
    template<typename T>
    static T convert(const Value& v, const std::string& name)
    {
        if (const T* p = std::get_if<T>(&v)) return *p;
        if constexpr (std::is_same_v<T, float>) {
            if (const int* i = std::get_if<int>(&v)) return static_cast<float>(*i);
        }
        if constexpr (std::is_same_v<T, bool>) {
            if (const int* i = std::get_if<int>(&v)) return *i != 0;
        }
        throw Error(__FILE__, __LINE__, __func__, "property \"" + name + "\" has another type");
    }

    std::map<std::string, Value> values_;
};

// ---------------------------------------------------------------- ground truth
// One labelled box, relative to the image (reference: GroundTruth, include/GroundTruth.h).
struct GroundTruth
{
    float x, y, w, h;
    int classId;
};

using GroundTruthVec = std::vector<GroundTruth>;

// ---------------------------------------------------------------- context
// The part of the owning model the layers read.
class Layer;

class Context
{
public:
    hipStream_t stream = nullptr;
    bool training = false;
    int width = 0, height = 0;      // network input size
    int classes = 0;

    // optimiser (reference: Model<D>::adam*, learningRate, momentum, decay, include/Model.h);
    // the shipped presets train with SGD + momentum (adam.enabled: False)
    bool adamEnabled = false;
    float learningRate = 1e-3f, momentum = 0.9f, decay = 5e-4f;
    float adamBeta1 = 0.9f, adamBeta2 = 0.999f, adamEpsilon = 1e-8f;
    int timeStep = 1;               // Adam's t
    int updateBatch = 1;            // images a parameter update averages over (batch * subdivisions)

    // The reference's update() rescales and clamps every layer's delta once more.  By then backward
    // has consumed it and the next forward clears it, so nothing reads the result; switching this
    // off drops one pass over every activation-sized tensor per step and changes no trained value.
    bool helpersTouchDeltaInUpdate = true;

    // Uploads the ground truth of the current batch: [batch][maxTruth][5] floats + counts.
    void setGroundTruth(const std::vector<GroundTruthVec>& batchTruth)
    {
        const auto batch = batchTruth.size();
        std::size_t most = 1;
        for (const auto& image: batchTruth) most = std::max(most, image.size());
        std::vector<float> packed(batch * most * 5, 0.0f);
        std::vector<int> counts(batch, 0);
        for (std::size_t b = 0; b < batch; ++b) {
            counts[b] = static_cast<int>(batchTruth[b].size());
            for (std::size_t t = 0; t < batchTruth[b].size(); ++t) {
                const auto& g = batchTruth[b][t];
                float* p = &packed[(b * most + t) * 5];
                p[0] = g.x; p[1] = g.y; p[2] = g.w; p[3] = g.h; p[4] = static_cast<float>(g.classId);
            }
        }
        if (truths_.size() != packed.size()) truths_ = FloatVector(packed.size());
        if (truthCounts_.size() != counts.size()) truthCounts_ = IntVector(counts.size());
        truths_.copyHost(packed, stream);
        truthCounts_.copyHost(counts, stream);
        maxTruth_ = static_cast<int>(most);
    }

    // One scratch buffer for the layers of this context.  They run one after the other on the
    // context's stream, so their uses cannot overlap, and another context (another model, another
    // stream) has a buffer of its own: nothing here goes through the library's shared per-device
    // workspace.  Layers reserve what their kernels need when they are constructed, so the buffer has
    // its final size and address before the first forward -- and before any graph capture.  A block
    // that has been outgrown is kept until the context goes, for graphs captured with its address.
    // Growing allocates and fills: an error while the context's stream is being captured (the constructors'
    // reservations are the growth path; a capture must find the buffer at its final size).
    void reserveWorkspace(std::size_t bytes)
    {
        if (bytes <= workspaceBytes()) return;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        const hipError_t asked = hipStreamIsCapturing(stream, &capturing);
        if (asked != hipSuccess) (void) hipGetLastError();
        PX_CHECK(asked == hipSuccess && capturing == hipStreamCaptureStatusNone,
                 "the context's workspace cannot grow while its stream is being captured: construct every layer "
                 "(or call reserveWorkspace) before the capture");
        // at least doubled, so that the retired blocks add up to less than the live one
        const std::size_t floats = std::max((bytes + sizeof(float) - 1) / sizeof(float), 2 * workspace_.size());
        if (!workspace_.empty()) retiredWorkspaces_.push_back(std::move(workspace_));
        workspace_ = FloatVector(floats, 0.0f, stream);
    }

    void* workspace() noexcept { return workspace_.empty() ? nullptr : workspace_.data(); }
    std::size_t workspaceBytes() const noexcept { return workspace_.size() * sizeof(float); }

    // Norm + peak from the kernel that wrote a delta (pxh_shortcut_backward_norm, pxh_axpy_norm): the
    // writer notes where it left the tensor's group sums, and the rescaleAndClip() that opens the
    // backward of the tensor's layer takes the note and starts from them instead of reading the
    // tensor.  A note is good for one use, and only if nothing writes the tensor in between: the
    // layers that leave one do so on request ("leaves_norm"), and whoever asks vouches for that.
    void noteNormGroups(const float* tensor, const float* groups) { normGroups_[tensor] = groups; }

    bool hasNormGroups(const float* tensor) const { return normGroups_.count(tensor) != 0; }

    const float* takeNormGroups(const float* tensor)
    {
        const auto it = normGroups_.find(tensor);
        if (it == normGroups_.end()) return nullptr;
        const float* groups = it->second;
        normGroups_.erase(it);
        return groups;
    }

    // YOLO heads that put their training forward off until the model's forward pass is over ("deferred"),
    // in the order they were reached: nothing reads a head's delta, cost or statistics before backward,
    // so all of them run as ONE pass then (YoloLayer::forwardDeferred), the small ones under the class
    // rows of the large one.  What they need of the context's workspace adds up, head by head.
    std::vector<Layer*> deferredHeads;
    std::size_t deferredHeadsWorkspace = 0;

    const FloatVector& truths() const noexcept { return truths_; }
    const IntVector& truthCounts() const noexcept { return truthCounts_; }
    int maxTruth() const noexcept { return maxTruth_; }

private:
    FloatVector truths_;
    IntVector truthCounts_;
    int maxTruth_ = 0;
    FloatVector workspace_;
    std::vector<FloatVector> retiredWorkspaces_;
    std::unordered_map<const float*, const float*> normGroups_;
};

// ---------------------------------------------------------------- layer
class ParameterSet;

class Layer
{
public:
    using V = FloatVector;
    using Ptr = std::shared_ptr<Layer>;

    Layer(Context& context, const Properties& props) : context_(context), props_(props)
    {
        batch_ = props.get<int>("batch", 1);
        channels_ = props.get<int>("channels", 3);
        height_ = props.get<int>("height", 0);
        width_ = props.get<int>("width", 0);
        index_ = props.get<int>("index", 0);
        inputs_ = props.get<int>("inputs", channels_ * height_ * width_);
        PX_CHECK(batch_ > 0 && channels_ > 0 && height_ >= 0 && width_ >= 0, "layer dimensions must be positive");
        if (context.training) context.reserveWorkspace(pxh_rescale_workspace_bytes());     // rescaleAndClip()
    }

    virtual ~Layer() = default;

    // Clears the per-pass state.  Derived classes call it first, as in the reference
    // (include/Layer.h:377-383), then write output_.
    virtual void forward(const V& /*input*/)
    {
        if (training() && !delta_.empty() && !firstConsumerOverwrites_) delta_.fill(0.0f, stream());
        cost_ = 0.0f;
    }

    // delta_ holds dL/d(output) on entry; a layer turns it into dL/d(input) and ACCUMULATES that
    // into *grad (nullptr for the first layer).
    // First the reference's two helpers on delta_ (include/Layer.h:385-397): rescale to a norm
    // threshold, then clamp; one fused call here.
    virtual void backward(const V& /*input*/, V* /*grad*/) { rescaleAndClip(delta_); }

    // The reference's update() runs the same two helpers once more, through the hooks that layers
    // with parameters extend to their update buffers (include/Layer.h:400-411, 473-493).  Derived
    // classes call this first, then rescaleAndClip() on each of their update tensors.
    virtual void update()
    {
        if (context_.helpersTouchDeltaInUpdate) rescaleAndClip(delta_);
    }

    // For a model that updates all its layers together (ParameterSet.h): a layer adds what its update()
    // works on to the set -- its delta here, its parameter tensors in the classes that have them (which
    // call this one first) -- and is told when the set has stepped them.
    virtual void collectParameters(ParameterSet& set);
    virtual void parametersUpdated() {}

    // This layer's section of a weight file; bytes read / written (reference: Layer<D>::loadWeights /
    // saveWeights, include/Layer.h:57-58).  Layers without parameters have none.
    virtual std::streamoff loadWeights(std::istream& /*is*/) { return 0; }
    virtual std::streamoff saveWeights(std::ostream& /*os*/) { return 0; }

    // Optimizer moments for the checkpoint sidecar; bytes written / read (reference:
    // Layer<D>::saveOptimizer / loadOptimizer, include/Layer.h:59-60).  Nothing by default.
    virtual std::streamoff saveOptimizer(std::ostream& /*os*/) { return 0; }
    virtual std::streamoff loadOptimizer(std::istream& /*is*/) { return 0; }

    virtual bool hasCost() const noexcept { return false; }
    float cost() const noexcept { return cost_; }

    int batch() const noexcept { return batch_; }
    int channels() const noexcept { return channels_; }
    int height() const noexcept { return height_; }
    int width() const noexcept { return width_; }
    int index() const noexcept { return index_; }
    int inputs() const noexcept { return inputs_; }
    int outChannels() const noexcept { return outChannels_; }
    int outHeight() const noexcept { return outHeight_; }
    int outWidth() const noexcept { return outWidth_; }
    int outputs() const noexcept { return outputs_; }

    const V& output() const noexcept { return output_; }
    V& delta() noexcept { return delta_; }

    // A layer whose delta is OVERWRITTEN by the first of its readers to run backward (a shortcut with
    // "first_writer") needs no zero-fill in forward.  Whoever sets this vouches that every backward
    // pass starts with that reader.
    void setFirstConsumerOverwrites(bool on) noexcept { firstConsumerOverwrites_ = on; }
    bool firstConsumerOverwrites() const noexcept { return firstConsumerOverwrites_; }

    void setGradientClipping(bool on, float value) { gradientClipping_ = on; gradientClipValue_ = value; }
    // thresholds of the two helpers as they apply to this layer's tensors; 0 = off
    float rescaleThreshold() const noexcept { return gradientRescaling_ ? gradientThreshold_ : 0.0f; }
    float clipValue() const noexcept { return gradientClipping_ ? gradientClipValue_ : 0.0f; }
    void setGradientRescaling(bool on, float threshold) { gradientRescaling_ = on; gradientThreshold_ = threshold; }

protected:
    // Sets the output shape and allocates output_ (and delta_, which inference never touches,
    // only when the context trains).
    void setOutput(int channels, int height, int width)
    {
        outChannels_ = channels;
        outHeight_ = height;
        outWidth_ = width;
        outputs_ = channels * height * width;
        const auto n = static_cast<std::size_t>(batch_) * outputs_;
        PX_CHECK(n < (std::size_t(1) << 31), "tensors of 2^31 elements or more are not supported");
        output_ = V(n);
        if (context_.training) delta_ = V(n);
    }

    // scaleTensor then constrain on one tensor, when the layer's flags ask for them; one fused call
    // that reads the tensor once and rewrites it only if some value has to change.
    // Where the kernel that wrote the tensor left its norm and peak behind (Context::noteNormGroups),
    // the tensor is not read at all unless it has to change; the result is the same to the bit.
    void rescaleAndClip(V& tensor)
    {
        if (tensor.empty()) return;
        const float* groups = context_.takeNormGroups(tensor.data());
        if (!(gradientRescaling_ || gradientClipping_)) return;
        context_.reserveWorkspace(pxh_rescale_workspace_bytes());
        const float threshold = gradientRescaling_ ? gradientThreshold_ : 0.0f;
        const float clip = gradientClipping_ ? gradientClipValue_ : 0.0f;
        if (groups)
            PX_HIP_CHECK(pxh_rescale_clip_from_groups(tensor.data(), tensor.size(), threshold, clip, nullptr, groups,
                                                      context_.workspace(), context_.workspaceBytes(), stream()));
        else
            PX_HIP_CHECK(pxh_rescale_clip(tensor.data(), tensor.size(), threshold, clip, nullptr, context_.workspace(),
                                          context_.workspaceBytes(), stream()));
    }

    // For a layer that leaves the norm of the delta in front of it behind ("leaves_norm"): the buffer
    // of group sums for a tensor of n values, allocated when the layer is built.
    static V normGroupsFor(std::size_t n) { return V((pxh_norm_groups_bytes(n) + sizeof(float) - 1) / sizeof(float)); }

    void checkInput(const V& input, const char* who) const
    {
        PX_CHECK(input.size() == static_cast<std::size_t>(batch_) * inputs_,
                 std::string(who) + ": input size does not match batch * inputs");
    }

    Context& context() noexcept { return context_; }
    const Context& context() const noexcept { return context_; }
    const Properties& properties() const noexcept { return props_; }
    hipStream_t stream() const noexcept { return context_.stream; }
    bool training() const noexcept { return context_.training; }
    bool inferring() const noexcept { return !context_.training; }

    V output_, delta_;
    float cost_ = 0.0f;

private:
    Context& context_;
    Properties props_;
    int batch_, channels_, height_, width_, index_, inputs_;
    int outChannels_ = 0, outHeight_ = 0, outWidth_ = 0, outputs_ = 0;
    bool gradientClipping_ = false, gradientRescaling_ = false, firstConsumerOverwrites_ = false;
    float gradientClipValue_ = 1.0f, gradientThreshold_ = 0.0f;
};

}   // px::hip
