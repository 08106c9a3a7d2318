// include/hip_lean/ModelExtras.h -- DeviceExtras<Device::HIP>, the model-wide state of the lean forms (the
// engine's DeviceExtras<Device::CUDA>, include/Model.h:101-127, holds the cuBLAS and cuDNN contexts in the same
// place).  Six things that a layer cannot know by itself:
//   * which deltas are OVERWRITTEN by the first backward that reaches them (a residual block's shortcut is the
//     first to write the delta of the layer in front of it and of its `from` layer): Layer::forward need not
//     clear those, and the shortcut writes instead of adding (pxh_shortcut_backward_first);
//   * where the kernel that wrote a delta last left the delta's norm and peak (pxh_shortcut_backward_norm,
//     pxh_axpy_norm): the rescale + clip that opens that layer's backward then reads 8 bytes per 256 values
//     instead of the tensor (pxh_rescale_clip_from_groups);
//   * which shortcuts ride on the epilogue of the convolution in front of them (pxh_bn_train_act_shortcut_forward);
//   * which max-pools do, at inference (pxh_bn_folded_act_maxpool_forward);
//   * the YOLO heads that wait for the end of the forward pass to run as one pass
//     (pxh_yolo_forward_train_heads);
//   * every layer's parameter tensors, as tables kept on the device: the update hooks and the optimiser step
//     of the whole model are three launches (pxh_rescale_clip_table, pxh_adam_update_table / pxh_sgd_update_table)
//     instead of ten per convolution.
// All of it leaves the values the plain bodies under include/hip/ leave, to the bit.
#pragma once

#include <map>
#include <set>
#include <vector>

#include "../hip/HipError.h"

namespace px {

template<>
class DeviceExtras<Device::HIP>
{
public:
    // ---- deltas whose first backward consumer overwrites them (marked once, when the graph is built)
    void markOverwritten(const float* delta) const { overwritten_.insert(delta); }
    bool overwritten(const float* delta) const { return overwritten_.count(delta) != 0; }

    // ---- norm + peak left behind by the kernel that wrote a delta last; a note is good for one use
    PxHipVector& normGroupsFor(const void* owner, std::size_t values) const
    {
        auto& g = groups_[owner];
        const std::size_t need = pxh_norm_groups_bytes(values) / sizeof(float);
        if (g.size() < need) g = PxHipVector(need);
        return g;
    }
    void noteNormGroups(const float* delta, const float* groups) const { notes_[delta] = groups; }
    bool hasNormGroups(const float* delta) const { return notes_.count(delta) != 0; }
    const float* takeNormGroups(const float* delta) const
    {
        const auto it = notes_.find(delta);
        if (it == notes_.end()) return nullptr;
        const float* groups = it->second;
        notes_.erase(it);
        return groups;
    }

    // ---- shortcuts that ride on the epilogue of the convolution in front of them (marked once, when the graph
    // is built, where nothing but the shortcut reads that convolution's output, the shortcut is linear over
    // tensors of one shape and its alpha is 1): the convolution writes the shortcut's output and works on the
    // shortcut's delta; the convolution's own delta is marked overwritten, it is never used
    struct Rider {
        PxHipVector* output;
        PxHipVector* delta;
        const PxHipVector* from;
        float alpha, beta;
    };
    void carry(const void* conv, const void* shortcut, const Rider& rider) const
    {
        riders_[conv] = rider;
        riding_.insert(shortcut);
    }
    const Rider* riderOf(const void* conv) const
    {
        const auto it = riders_.find(conv);
        return it == riders_.end() ? nullptr : &it->second;
    }
    bool rides(const void* layer) const { return riding_.count(layer) != 0; }

    // ---- max-pools that ride on the epilogue of the convolution in front of them, at inference (the 2 x 2 window
    // at stride 2 over planes of even size): the convolution writes the pool's output; its own only when
    // something else reads it as well (`keepOutput`: a route names the convolution)
    struct PoolRider {
        PxHipVector* pooled;
        bool keepOutput;
    };
    void carryPool(const void* conv, const void* pool, const PoolRider& rider) const
    {
        poolRiders_[conv] = rider;
        riding_.insert(pool);
    }
    const PoolRider* poolOf(const void* conv) const
    {
        const auto it = poolRiders_.find(conv);
        return it == poolRiders_.end() ? nullptr : &it->second;
    }

    // ---- YOLO heads waiting for the end of the forward pass
    struct WaitingHead {
        pxh_yolo_head head;
        const int* anchors;
        int anchorCount, batch, classes;
        const float* truths;
        const int* truthCounts;
        int maxTruth;
    };
    void deferHead(const WaitingHead& h) const { waiting_.push_back(h); }

    // after the last layer's forward (Model<D>::forward, include/Model.h:1740-1759): all waiting heads, one pass
    void forwardDeferredHeads(int netWidth, int netHeight) const
    {
        std::vector<pxh_yolo_head> heads;
        for (std::size_t first = 0; first < waiting_.size(); first += 4) {
            heads.clear();
            for (std::size_t h = first; h < waiting_.size() && h < first + 4; ++h) heads.push_back(waiting_[h].head);
            const auto& w = waiting_[first];
            PX_HIP_CHECK(pxh_yolo_forward_train_heads(static_cast<int>(heads.size()), heads.data(), w.truths, w.truthCounts,
                                                      w.maxTruth, w.anchors, w.anchorCount, w.batch, w.classes, netWidth,
                                                      netHeight, nullptr, 0, nullptr));
        }
        waiting_.clear();
    }

    // ---- parameter tensors of all layers: weights / updates / first / second moments, side by side
    void registerParameters(PxHipVector& w, PxHipVector& updates, PxHipVector& m, PxHipVector& v, bool decayed) const
    {
        if (w.size() == 0) return;
        tensors_[0].push_back(w.data()); tensors_[1].push_back(updates.data());
        tensors_[2].push_back(m.size() ? m.data() : nullptr); tensors_[3].push_back(v.size() ? v.data() : nullptr);
        sizes_.push_back(w.size());
        decayed_.push_back(decayed ? 1 : 0);
        dropTables();
    }

    // Model<D>::update (include/Model.h:1784-1792) for all layers at once: the two gradient hooks on every update
    // buffer (each buffer with its own norm, as Layer::scaleTensor gives it), then the optimiser step.
    void updateAll(bool rescale, float threshold, bool clip, float clipValue, bool adam, int batch, int t, float lr,
                   float momentum, float beta1, float beta2, float epsilon, float decay) const
    {
        if (sizes_.empty()) return;
        if (!hooks_) {
            float* const* only[1] = { tensors_[1].data() };
            PX_HIP_CHECK(pxh_tensor_table_create(static_cast<int>(sizes_.size()), 1, only[0], sizes_.data(), nullptr, &hooks_));
            std::vector<float*> flat;
            const int streams = adam ? 4 : 2;
            for (int s = 0; s < streams; ++s) flat.insert(flat.end(), tensors_[s].begin(), tensors_[s].end());
            PX_HIP_CHECK(pxh_tensor_table_create(static_cast<int>(sizes_.size()), streams, flat.data(), sizes_.data(),
                                                 decayed_.data(), &step_));
        }
        if (rescale || clip)
            PX_HIP_CHECK(pxh_rescale_clip_table(hooks_, rescale ? threshold : 0.0f, clip ? clipValue : 0.0f, nullptr, nullptr));
        if (adam) PX_HIP_CHECK(pxh_adam_update_table(step_, batch, t, lr, beta1, beta2, epsilon, decay, nullptr));
        else PX_HIP_CHECK(pxh_sgd_update_table(step_, batch, lr, momentum, decay, nullptr));
    }

    ~DeviceExtras() { dropTables(); }

private:
    void dropTables() const
    {
        if (hooks_) pxh_tensor_table_destroy(hooks_);
        if (step_) pxh_tensor_table_destroy(step_);
        hooks_ = step_ = nullptr;
    }

    mutable std::set<const float*> overwritten_;
    mutable std::map<const void*, PxHipVector> groups_;
    mutable std::map<const float*, const float*> notes_;
    mutable std::map<const void*, Rider> riders_;
    mutable std::map<const void*, PoolRider> poolRiders_;
    mutable std::set<const void*> riding_;
    mutable std::vector<WaitingHead> waiting_;
    mutable std::vector<float*> tensors_[4];
    mutable std::vector<std::size_t> sizes_;
    mutable std::vector<int> decayed_;
    mutable pxh_tensor_table* hooks_ = nullptr;
    mutable pxh_tensor_table* step_ = nullptr;
};

}   // px
