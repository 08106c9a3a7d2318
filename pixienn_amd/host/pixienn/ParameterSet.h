// The parameter tensors of a model, gathered once, updated together.
//
// The reference updates layer by layer (Model<D>::update, include/Model.h:1786-1792): per convolution
// the scaleGradients / clipGradients hooks on three update buffers and three optimiser calls
// (include/ConvLayer.h:299-340, include/cuda/ConvLayer.h:362-413).  Most of those tensors are a few
// hundred values, so on the GPU that loop is a thousand launches that each take longer to start than to
// run.  A ParameterSet holds the same tensors and does the same arithmetic on each of them through
// tables of tensors kept on the device (pxh_tensor_table_*), built the first time the set is stepped: the
// optimiser is ONE launch for all tensors, the hooks two per pair of thresholds:
//
//     ParameterSet params;
//     for (auto& layer: layers) layer->collectParameters(params);      // once, after construction
//     ...
//     params.update(context);                  // instead of every layer's update(): hooks + optimiser
//     for (auto& layer: layers) layer->parametersUpdated();
//
// Every tensor ends up bit for bit as its layer's own update() leaves it -- the deltas included, which
// the reference's update() passes through the two helpers once more (Context::helpersTouchDeltaInUpdate).
#pragma once

#include <map>
#include <utility>
#include <vector>

#include "Layer.h"

namespace px::hip {

// Owning handle of a pxh_tensor_table (move-only).
class TensorTable
{
public:
    TensorTable() = default;

    // `streams` buffer lists of `count` tensors each, stream after stream
    TensorTable(int count, int streams, const std::vector<float*>& buffers, const std::vector<std::size_t>& n,
                const std::vector<int>* decayed)
    {
        PX_HIP_CHECK(pxh_tensor_table_create(count, streams, buffers.data(), n.data(), decayed ? decayed->data() : nullptr,
                                             &table_));
    }

    TensorTable(const TensorTable&) = delete;
    TensorTable& operator=(const TensorTable&) = delete;
    TensorTable(TensorTable&& rhs) noexcept : table_(rhs.table_) { rhs.table_ = nullptr; }

    TensorTable& operator=(TensorTable&& rhs) noexcept
    {
        if (this != &rhs) {
            pxh_tensor_table_destroy(table_);
            table_ = rhs.table_;
            rhs.table_ = nullptr;
        }
        return *this;
    }

    ~TensorTable() { pxh_tensor_table_destroy(table_); }

    const pxh_tensor_table* get() const noexcept { return table_; }
    explicit operator bool() const noexcept { return table_ != nullptr; }

private:
    pxh_tensor_table* table_ = nullptr;
};

class ParameterSet
{
public:
    using V = FloatVector;

    // thresholds of the two hooks for a tensor's update buffer; 0 = hook off
    struct Hooks {
        float rescaleThreshold = 0.0f, clipValue = 0.0f;
    };

    // values, their accumulated update, Adam's two moments; `decayed`: takes the weight decay
    void addAdam(V& w, V& d, V& m, V& v, bool decayed, Hooks hooks)
    {
        if (w.empty()) return;
        PX_CHECK(w.size() == d.size() && w.size() == m.size() && w.size() == v.size(),
                 "ParameterSet: tensors of different sizes");
        adam_.add(w, d, decayed);
        adam_.m.push_back(m.data());
        adam_.v.push_back(v.data());
        hook(d, hooks);
        built_ = false;
    }

    // values and their accumulated update (which becomes the momentum term)
    void addSgd(V& w, V& d, bool decayed, Hooks hooks)
    {
        if (w.empty()) return;
        PX_CHECK(w.size() == d.size(), "ParameterSet: tensors of different sizes");
        sgd_.add(w, d, decayed);
        hook(d, hooks);
        built_ = false;
    }

    // a layer's delta, for the helpers' pass over it in update()
    void addDelta(V& delta, Hooks hooks)
    {
        if (!delta.empty()) hook(delta, hooks);
        built_ = false;
    }

    // parameter tensors held (deltas not counted)
    std::size_t tensors() const noexcept { return adam_.w.size() + sgd_.w.size(); }

    void clear() { *this = ParameterSet(); }

    ParameterSet() = default;
    ParameterSet(ParameterSet&&) = default;
    ParameterSet& operator=(ParameterSet&&) = default;

    // Builds the device tables of what has been added (allocates and uploads: not under graph capture).
    // update() does it by itself the first time; a model that captures its update calls this first.
    void build()
    {
        if (built_) return;
        adamTable_ = TensorTable();
        sgdTable_ = TensorTable();
        for (auto& [key, group]: hooked_) group.table = TensorTable();
        if (!adam_.w.empty()) {
            std::vector<float*> buffers(adam_.w);
            buffers.insert(buffers.end(), adam_.d.begin(), adam_.d.end());
            buffers.insert(buffers.end(), adam_.m.begin(), adam_.m.end());
            buffers.insert(buffers.end(), adam_.v.begin(), adam_.v.end());
            adamTable_ = TensorTable(static_cast<int>(adam_.w.size()), 4, buffers, adam_.n, &adam_.decayed);
        }
        if (!sgd_.w.empty()) {
            std::vector<float*> buffers(sgd_.w);
            buffers.insert(buffers.end(), sgd_.d.begin(), sgd_.d.end());
            sgdTable_ = TensorTable(static_cast<int>(sgd_.w.size()), 2, buffers, sgd_.n, &sgd_.decayed);
        }
        for (auto& [key, group]: hooked_)
            group.table = TensorTable(static_cast<int>(group.x.size()), 1, group.x, group.n, nullptr);
        built_ = true;
    }

    // The hooks on every update buffer, then the optimiser step, with the context's settings.
    void update(const Context& c)
    {
        build();
        for (const auto& [key, group]: hooked_)
            PX_HIP_CHECK(pxh_rescale_clip_table(group.table.get(), key.first, key.second, nullptr, c.stream));
        if (adamTable_) {
            PX_CHECK(c.updateBatch > 0 && c.timeStep > 0, "Adam needs batch > 0 and t > 0");
            PX_HIP_CHECK(pxh_adam_update_table(adamTable_.get(), c.updateBatch, c.timeStep, c.learningRate, c.adamBeta1,
                                               c.adamBeta2, c.adamEpsilon, c.decay, c.stream));
        }
        if (sgdTable_)
            PX_HIP_CHECK(pxh_sgd_update_table(sgdTable_.get(), c.updateBatch, c.learningRate, c.momentum, c.decay,
                                              c.stream));
    }

private:
    struct Group {
        std::vector<float*> w, d, m, v;
        std::vector<std::size_t> n;
        std::vector<int> decayed;
        void add(V& values, V& updates, bool decay)
        {
            w.push_back(values.data());
            d.push_back(updates.data());
            n.push_back(values.size());
            decayed.push_back(decay ? 1 : 0);
        }
    };
    struct Hooked {
        std::vector<float*> x;
        std::vector<std::size_t> n;
        TensorTable table;
    };

    void hook(V& updates, Hooks h)
    {
        if (!(h.rescaleThreshold > 0.0f) && !(h.clipValue > 0.0f)) return;
        Hooked& group = hooked_[{ h.rescaleThreshold, h.clipValue }];
        group.x.push_back(updates.data());
        group.n.push_back(updates.size());
    }

    Group adam_, sgd_;
    std::map<std::pair<float, float>, Hooked> hooked_;     // update buffers by (threshold, clip)
    TensorTable adamTable_, sgdTable_;
    bool built_ = false;
};

// what Layer::update() does, as an entry of the set
inline void Layer::collectParameters(ParameterSet& set)
{
    if (context_.helpersTouchDeltaInUpdate) set.addDelta(delta_, ParameterSet::Hooks{ rescaleThreshold(), clipValue() });
}

}  // namespace px::hip
