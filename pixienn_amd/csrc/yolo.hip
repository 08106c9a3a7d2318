// YOLO head for gfx950: logistic decode, and the training pass (decode + dense delta + cost +
// statistics) in one sweep over the head tensor.
//
// Layout [batch][mask][5 + classes][area]: for a fixed entry consecutive lanes hold consecutive
// cells, so every load and store of the sweep is a coalesced row segment.
// Box arithmetic follows the CPU layer (include/YoloLayer.h, src/DarkBox.cpp of the reference).
#include "stream.h"

#include <cfloat>

namespace pxh {
namespace {

constexpr int kMaxAnchors = 32;
constexpr int kMaxMasks = 16;
constexpr int kTruthTile = kBlock;
constexpr int kSums = 13;   // stats[12] + cost

// ---------------------------------------------------------------- boxes
struct Box { float x, y, w, h; };

// cv::Rect_<float>::operator& (OpenCV >= 4.5.4) on the top-left rectangles of two centre boxes,
// as DarkBox::intersection builds them (src/DarkBox.cpp:84-131).
__device__ __forceinline__ float box_intersection(const Box& a, const Box& b)
{
    if (a.w <= 0.0f || a.h <= 0.0f || b.w <= 0.0f || b.h <= 0.0f) return 0.0f;
    const float ax = a.x - a.w / 2.0f, ay = a.y - a.h / 2.0f;   // extents are positive here
    const float bx = b.x - b.w / 2.0f, by = b.y - b.h / 2.0f;
    const bool a_left = ax < bx, a_top = ay < by;
    const float xlo = a_left ? ax : bx, xlo_w = a_left ? a.w : b.w;
    const float xhi = a_left ? bx : ax, xhi_w = a_left ? b.w : a.w;
    const float ylo = a_top ? ay : by, ylo_h = a_top ? a.h : b.h;
    const float yhi = a_top ? by : ay, yhi_h = a_top ? b.h : a.h;
    if ((xlo < 0.0f && xlo + xlo_w < xhi) || (ylo < 0.0f && ylo + ylo_h < yhi)) return 0.0f;
    const float iw = fminf(xlo_w - (xhi - xlo), xhi_w);
    const float ih = fminf(ylo_h - (yhi - ylo), yhi_h);
    if (iw <= 0.0f || ih <= 0.0f) return 0.0f;
    return iw * ih;
}

__device__ __forceinline__ float box_iou(const Box& a, const Box& b)
{
    const float inter = box_intersection(a, b);
    const float aa = a.w * a.h;
    const float ab = b.w * b.h;
    float uni = aa + ab;
    uni = uni - inter;
    uni = uni > 0.0f ? uni : 0.0f;
    if (uni == 0.0f) return 0.0f;
    return inter / uni;
}

// ---------------------------------------------------------------- decode only
struct YoloActivateOp {
    const float* in;
    float* out;
    FastDiv by_area;
    FastDiv by_entries;
    template<int V> struct Regs { Pack<V> x; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const { r.x = ld<V, NT>(in, e); }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        uint32_t plane, off, q, entry;
        by_area.divmod(static_cast<uint32_t>(e), plane, off);
        by_entries.divmod(plane, q, entry);
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            if (off + k >= by_area.d) {   // next row of the [entries][area] matrix
                off -= by_area.d;
                entry = entry + 1 == by_entries.d ? 0 : entry + 1;
            }
            const float x = r.x.v[k];
            o.v[k] = (entry < 2 || entry >= 4) ? 1.0f / (1.0f + expf(-x)) : x;
        }
        st<V, NT>(out, e, o);
    }
};

// ---------------------------------------------------------------- training sweep
struct YoloParams {
    int batch, mask_count, anchor_count, classes, width, height, area;
    int net_width, net_height, max_truth;
    float ignore_thresh, truth_thresh, coord_scale, object_scale, noobject_scale, class_scale;
    int masks[kMaxMasks];
    float anchors[2 * kMaxAnchors];   // integer pixel sizes held as float
    FastDiv by_tiles;
    FastDiv by_masks;
    FastDiv by_width;
};

// Tables of the reference's signature (host-built assignment), all device pointers.
struct YoloTables {
    const int* assigned_classes;
    const int* assigned_anchors;
    const float* assigned_boxes;
    const int* masks;
    const float* anchors;
};

struct TruthSlot {
    Box box;
    int cls;
    int target;   // mask_slot * area + cell of the positive this truth claims, or -1
    int anchor;   // its best anchor over all anchors
};

__device__ __forceinline__ Box decode_box(float sx, float sy, float rw, float rh, int i, int j, float aw, float ah,
                                          const YoloParams& p)
{
    Box b;
    b.x = (static_cast<float>(i) + sx) / static_cast<float>(p.width);
    b.y = (static_cast<float>(j) + sy) / static_cast<float>(p.height);
    b.w = expf(rw) * aw / static_cast<float>(p.net_width);
    b.h = expf(rh) * ah / static_cast<float>(p.net_height);
    return b;
}

struct BoxDelta { float v[4]; };

// include/YoloLayer.h:408-436
__device__ __forceinline__ BoxDelta box_delta(const Box& truth, float sx, float sy, float rw, float rh, int i, int j,
                                              float aw, float ah, const YoloParams& p)
{
    const float tx = truth.x * static_cast<float>(p.width) - static_cast<float>(i);
    const float ty = truth.y * static_cast<float>(p.height) - static_cast<float>(j);
    const float tw = logf(fmaxf(1e-9f, truth.w * static_cast<float>(p.net_width) / aw));
    const float th = logf(fmaxf(1e-9f, truth.h * static_cast<float>(p.net_height) / ah));
    const float scale = p.coord_scale * (2.0f - truth.w * truth.h);
    BoxDelta d;
    d.v[0] = scale * (tx - sx);
    d.v[1] = scale * (ty - sy);
    d.v[2] = scale * (tw - rw);
    d.v[3] = scale * (th - rh);
    return d;
}

// FUSED: raw logits in, decode written to `out`, positives found from the truths on the device
//        with the CPU layer's rule; statistics as the CPU layer accumulates them.
// !FUSED: `in` is the already decoded head, positives come from the host-built tables;
//        statistics as the reference's device path accumulates them.
template<bool FUSED>
__global__ __launch_bounds__(kBlock) void yolo_train_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                            float* __restrict__ delta,
                                                            const float* __restrict__ truths,
                                                            const int* __restrict__ truth_counts, YoloParams p,
                                                            YoloTables tb, double* __restrict__ partial)
{
    __shared__ TruthSlot tile[kTruthTile];
    __shared__ double slots[kBlock / kWave];

    uint32_t bn, tile_id, b, n;
    p.by_tiles.divmod(blockIdx.x, bn, tile_id);
    p.by_masks.divmod(bn, b, n);
    const int cell = tile_id * kBlock + threadIdx.x;
    const bool live = cell < p.area;
    const int area = p.area;
    const int entries = p.classes + 5;
    const size_t base = (static_cast<size_t>(bn) * entries) * area + (live ? cell : 0);

    int mask_anchor;
    float aw, ah;
    if constexpr (FUSED) {
        mask_anchor = p.masks[n];
        aw = p.anchors[2 * mask_anchor];
        ah = p.anchors[2 * mask_anchor + 1];
    } else {
        mask_anchor = tb.masks[n];
        aw = tb.anchors[2 * mask_anchor];
        ah = tb.anchors[2 * mask_anchor + 1];
    }

    uint32_t row, col;
    p.by_width.divmod(live ? cell : 0, row, col);
    const int i = col, j = row;

    // head entries 0..4
    float sx = 0, sy = 0, rw = 0, rh = 0, so = 0;
    if (live) {
        const float v0 = in[base], v1 = in[base + area], v2 = in[base + 2 * static_cast<size_t>(area)],
                    v3 = in[base + 3 * static_cast<size_t>(area)], v4 = in[base + 4 * static_cast<size_t>(area)];
        if constexpr (FUSED) {
            sx = 1.0f / (1.0f + expf(-v0));
            sy = 1.0f / (1.0f + expf(-v1));
            so = 1.0f / (1.0f + expf(-v4));
            out[base] = sx;
            out[base + area] = sy;
            out[base + 2 * static_cast<size_t>(area)] = v2;
            out[base + 3 * static_cast<size_t>(area)] = v3;
            out[base + 4 * static_cast<size_t>(area)] = so;
        } else {
            sx = v0; sy = v1; so = v4;
        }
        rw = v2; rh = v3;
    }
    const Box pred = decode_box(sx, sy, rw, rh, i, j, aw, ah, p);

    // sweep the image's truths through LDS: best IoU (strict >, first wins) and, in the fused
    // form, the truths that claim this slot as their positive (the last one writes the delta).
    const int count = truth_counts[b];
    float best = -FLT_MAX;
    int best_cls = -1;
    Box best_box{ 0, 0, 0, 0 };
    bool have_best = false;
    int pos_cls = -1, pos_anchor = mask_anchor;
    Box pos_box{ 0, 0, 0, 0 };
    float st_iou = 0, st_r50 = 0, st_r75 = 0, st_cat = 0, st_obj = 0, st_count = 0;
    const int my_slot = n * area + cell;

    for (int t0 = 0; t0 < count; t0 += kTruthTile) {
        const int t = t0 + threadIdx.x;
        __syncthreads();
        if (t < count) {
            const float* g = truths + (static_cast<size_t>(b) * p.max_truth + t) * 5;
            TruthSlot s;
            s.box = Box{ g[0], g[1], g[2], g[3] };
            s.cls = static_cast<int>(g[4]);
            s.target = -1;
            s.anchor = 0;
            if constexpr (FUSED) {
                // best anchor over all anchors against the origin-shifted truth
                const Box shifted{ 0.0f, 0.0f, s.box.w, s.box.h };
                float ba = -FLT_MAX;
                int bi = 0;
                for (int a = 0; a < p.anchor_count; ++a) {
                    const Box cand{ 0.0f, 0.0f, p.anchors[2 * a] / static_cast<float>(p.net_width),
                                    p.anchors[2 * a + 1] / static_cast<float>(p.net_height) };
                    const float iou = box_iou(cand, shifted);
                    if (iou > ba) { ba = iou; bi = a; }
                }
                int ms = -1;
                for (int m = 0; m < p.mask_count; ++m)
                    if (p.masks[m] == bi) { ms = m; break; }
                if (ms >= 0) {
                    int ci = static_cast<int>(s.box.x * static_cast<float>(p.width));
                    int cj = static_cast<int>(s.box.y * static_cast<float>(p.height));
                    ci = max(0, min(ci, p.width - 1));
                    cj = max(0, min(cj, p.height - 1));
                    s.target = ms * area + cj * p.width + ci;
                    s.anchor = bi;
                }
            }
            tile[threadIdx.x] = s;
        }
        __syncthreads();
        const int tn = min(kTruthTile, count - t0);
        if (live) {
            for (int k = 0; k < tn; ++k) {
                const TruthSlot s = tile[k];
                const float iou = box_iou(pred, s.box);
                if (iou > best) {
                    best = iou;
                    best_cls = s.cls;
                    best_box = s.box;
                    have_best = true;
                }
                if constexpr (FUSED) {
                    if (s.target == my_slot) {
                        // every claiming truth is counted (include/YoloLayer.h:480-507); s.anchor is
                        // this mask's anchor, so `iou` above is the IoU the CPU layer records
                        pos_cls = s.cls;
                        pos_box = s.box;
                        pos_anchor = s.anchor;
                        const float logit = in[base + (5 + static_cast<size_t>(s.cls)) * area];
                        st_cat += fminf(1.0f, 1.0f / (1.0f + expf(-logit)));
                        st_iou += iou;
                        if (iou > .5f) st_r50 += 1.0f;
                        if (iou > .75f) st_r75 += 1.0f;
                        st_obj += so;
                        st_count += 1.0f;
                    }
                }
            }
        }
    }

    if constexpr (!FUSED) {
        if (live) {
            const size_t slot = static_cast<size_t>(bn) * area + cell;
            const int cls = tb.assigned_classes[slot];
            if (cls >= 0) {
                pos_cls = cls;
                pos_anchor = tb.assigned_anchors[slot];
                const float* bx = tb.assigned_boxes + slot * 4;
                pos_box = Box{ bx[0], bx[1], bx[2], bx[3] };
                const float paw = tb.anchors[2 * pos_anchor], pah = tb.anchors[2 * pos_anchor + 1];
                const float iou = box_iou(decode_box(sx, sy, rw, rh, i, j, paw, pah, p), pos_box);
                st_iou = iou;
                st_r50 = iou > .5f ? 1.0f : 0.0f;
                st_r75 = iou > .75f ? 1.0f : 0.0f;
                st_obj = so;
                st_count = 1.0f;
                st_cat = fminf(1.0f, in[base + (5 + static_cast<size_t>(cls)) * area]);
            }
        }
    }

    // region decision (include/YoloLayer.h:531-545), then the positive override (480-497)
    float d_obj = 0.0f;
    int cls = -1;            // class the dense class delta is written for, -1: zeros
    BoxDelta bd{ { 0, 0, 0, 0 } };
    if (live) {
        if (!have_best || best < p.ignore_thresh) d_obj = p.noobject_scale * (0.0f - so);
        if (have_best && best > p.truth_thresh) {
            d_obj = p.object_scale * (1.0f - so);
            cls = best_cls;
            bd = box_delta(best_box, sx, sy, rw, rh, i, j, aw, ah, p);
            if constexpr (FUSED) {
                // deltaYoloClass also feeds the class-probability statistic on this path
                const float logit = in[base + (5 + static_cast<size_t>(best_cls)) * area];
                st_cat += fminf(1.0f, 1.0f / (1.0f + expf(-logit)));
            }
        }
        if (pos_cls >= 0) {
            float paw = aw, pah = ah;
            if constexpr (!FUSED) {
                paw = tb.anchors[2 * pos_anchor];
                pah = tb.anchors[2 * pos_anchor + 1];
            }
            bd = box_delta(pos_box, sx, sy, rw, rh, i, j, paw, pah, p);
            d_obj = p.object_scale * (1.0f - so);
            cls = pos_cls;
        }
    }

    float c_box = 0, c_obj = 0, c_noobj = 0, c_cls = 0;
    if (live) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            delta[base + k * static_cast<size_t>(area)] = bd.v[k];
            c_box += bd.v[k] * bd.v[k];
        }
        delta[base + 4 * static_cast<size_t>(area)] = d_obj;
        if (d_obj >= 0.0f) c_obj = d_obj * d_obj; else c_noobj = d_obj * d_obj;

        // classes: decode (fused) and dense delta in one pass over the 'classes' rows
        const size_t cbase = base + 5 * static_cast<size_t>(area);
#pragma unroll 8
        for (int c = 0; c < p.classes; ++c) {
            const float v = in[cbase + c * static_cast<size_t>(area)];
            float prob = v;
            if constexpr (FUSED) {
                prob = 1.0f / (1.0f + expf(-v));
                out[cbase + c * static_cast<size_t>(area)] = prob;
            }
            float d = 0.0f;
            if (cls >= 0) {
                const float t = (c == cls) ? 1.0f : 0.0f;
                d = p.class_scale * (t - prob);
            }
            delta[cbase + c * static_cast<size_t>(area)] = d;
            c_cls += d * d;
        }
    }

    const double sums[kSums] = { st_iou, st_r50, st_r75, st_cat, st_obj, live ? so : 0.0f, st_count, st_count,
                                 c_box, c_obj, c_noobj, c_cls,
                                 static_cast<double>(c_box) + c_obj + c_noobj + c_cls };
#pragma unroll
    for (int k = 0; k < kSums; ++k) {
        const double total = block_sum(sums[k], slots);
        if (threadIdx.x == 0) partial[static_cast<size_t>(blockIdx.x) * kSums + k] = total;
    }
}

// One workgroup adds the per-workgroup sums in a fixed order.
__global__ __launch_bounds__(kBlock) void yolo_finish_kernel(const double* partial, int blocks, float* stats,
                                                             float* cost, int accumulate)
{
    __shared__ double slots[kBlock / kWave];
    for (int k = 0; k < kSums; ++k) {
        double s = 0.0;
        for (int j = threadIdx.x; j < blocks; j += kBlock) s += partial[static_cast<size_t>(j) * kSums + k];
        const double total = block_sum(s, slots);
        if (threadIdx.x == 0) {
            const float v = static_cast<float>(total);
            if (k < 12) {
                if (stats) stats[k] = (accumulate ? stats[k] : 0.0f) + v;
            } else if (cost) {
                *cost = (accumulate ? *cost : 0.0f) + v;
            }
        }
    }
}

int fill_params(const char* who, YoloParams& p, int batch, int mask_count, int anchor_count, int classes, int width,
                int height, int net_width, int net_height, int max_truth, float ignore_thresh, float truth_thresh,
                float coord_scale, float object_scale, float noobject_scale, float class_scale)
{
    if (batch <= 0 || mask_count <= 0 || anchor_count <= 0 || classes <= 0 || width <= 0 || height <= 0 ||
        net_width <= 0 || net_height <= 0 || max_truth < 0)
        return fail_invalid("%s: sizes must be positive", who);
    if (mask_count > kMaxMasks || anchor_count > kMaxAnchors) {
        set_error("%s: at most %d masks and %d anchors are supported", who, kMaxMasks, kMaxAnchors);
        return PXH_ERR_UNSUPPORTED;
    }
    const unsigned long long total = 1ull * batch * mask_count * (classes + 5) * width * height;
    if (total >= (1ull << 31)) {
        set_error("%s: tensors of 2^31 elements or more are not supported", who);
        return PXH_ERR_UNSUPPORTED;
    }
    p.batch = batch; p.mask_count = mask_count; p.anchor_count = anchor_count; p.classes = classes;
    p.width = width; p.height = height; p.area = width * height;
    p.net_width = net_width; p.net_height = net_height; p.max_truth = max_truth;
    p.ignore_thresh = ignore_thresh; p.truth_thresh = truth_thresh; p.coord_scale = coord_scale;
    p.object_scale = object_scale; p.noobject_scale = noobject_scale; p.class_scale = class_scale;
    const int tiles = (p.area + kBlock - 1) / kBlock;
    p.by_tiles = FastDiv(tiles);
    p.by_masks = FastDiv(mask_count);
    p.by_width = FastDiv(width);
    return PXH_OK;
}

int train_blocks(const YoloParams& p) { return p.batch * p.mask_count * static_cast<int>(p.by_tiles.d); }

}  // namespace
}  // namespace pxh

using namespace pxh;

extern "C" {

int pxh_yolo_activate(const float* input, float* output, int batch, int masks, int classes, int area, void* stream)
{
    if (!input || !output) return fail_invalid("pxh_yolo_activate: null pointer");
    if (batch <= 0 || masks <= 0 || classes < 0 || area <= 0) return fail_invalid("pxh_yolo_activate: sizes must be positive");
    const unsigned long long total = 1ull * batch * masks * (classes + 5) * area;
    if (total >= (1ull << 31)) {
        set_error("pxh_yolo_activate: tensors of 2^31 elements or more are not supported");
        return PXH_ERR_UNSUPPORTED;
    }
    YoloActivateOp op{ input, output, FastDiv(area), FastDiv(classes + 5) };
    // the 128-bit path steps a row boundary at most once per vector: needs area >= 4
    const bool vec = area >= 4 && aligned16(input) && aligned16(output);
    return launch_stream("pxh_yolo_activate", static_cast<size_t>(total), vec, 8, op, as_stream(stream));
}

size_t pxh_yolo_workspace_bytes(int batch, int mask_count, int classes, int width, int height)
{
    (void) classes;
    if (batch <= 0 || mask_count <= 0 || width <= 0 || height <= 0) return 0;
    const size_t tiles = (static_cast<size_t>(width) * height + kBlock - 1) / kBlock;
    return static_cast<size_t>(batch) * mask_count * tiles * kSums * sizeof(double);
}

int pxh_yolo_forward_train(const float* input, float* output, float* delta, const float* truths,
                           const int* truth_counts, int max_truth, const int* host_masks, const int* host_anchors,
                           float* stats, float* cost, int batch, int mask_count, int anchor_count, int classes,
                           int width, int height, int net_width, int net_height, float ignore_thresh,
                           float truth_thresh, float coord_scale, float object_scale, float noobject_scale,
                           float class_scale, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!input || !output || !delta || !truth_counts || !host_masks || !host_anchors || (!truths && max_truth > 0))
        return fail_invalid("pxh_yolo_forward_train: null pointer");
    if (input == output || input == delta || output == delta)
        return fail_invalid("pxh_yolo_forward_train: input, output and delta must be distinct buffers");
    YoloParams p{};
    int rc = fill_params("pxh_yolo_forward_train", p, batch, mask_count, anchor_count, classes, width, height,
                         net_width, net_height, max_truth, ignore_thresh, truth_thresh, coord_scale, object_scale,
                         noobject_scale, class_scale);
    if (rc) return rc;
    for (int m = 0; m < mask_count; ++m) {
        if (host_masks[m] < 0 || host_masks[m] >= anchor_count)
            return fail_invalid("pxh_yolo_forward_train: mask %d names anchor %d of %d", m, host_masks[m], anchor_count);
        p.masks[m] = host_masks[m];
    }
    for (int a = 0; a < 2 * anchor_count; ++a) p.anchors[a] = static_cast<float>(host_anchors[a]);
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes,
                           pxh_yolo_workspace_bytes(batch, mask_count, classes, width, height), &ws);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const int blocks = train_blocks(p);
    hipLaunchKernelGGL((yolo_train_kernel<true>), dim3(blocks), dim3(kBlock), 0, s, input, output, delta, truths,
                       truth_counts, p, YoloTables{}, static_cast<double*>(ws));
    rc = check_launch("yolo_train");
    if (rc) return rc;
    hipLaunchKernelGGL(yolo_finish_kernel, dim3(1), dim3(kBlock), 0, s, static_cast<const double*>(ws), blocks, stats,
                       cost, 0);
    return check_launch("yolo_finish");
}

int pxh_yolo_loss(const float* output, float* delta, const float* truths, const int* truth_counts, int max_truth,
                  const int* assigned_classes, const int* assigned_anchors, const float* assigned_boxes,
                  const int* masks, const float* anchors, float* stats, float* cost, int batch, int mask_count,
                  int anchor_count, int classes, int width, int height, int net_width, int net_height,
                  float ignore_thresh, float truth_thresh, float coord_scale, float object_scale,
                  float noobject_scale, float class_scale, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!output || !delta || !truth_counts || !assigned_classes || !assigned_anchors || !assigned_boxes || !masks ||
        !anchors || (!truths && max_truth > 0))
        return fail_invalid("pxh_yolo_loss: null pointer");
    if (output == delta) return fail_invalid("pxh_yolo_loss: output and delta must be distinct buffers");
    YoloParams p{};
    int rc = fill_params("pxh_yolo_loss", p, batch, mask_count, anchor_count, classes, width, height, net_width,
                         net_height, max_truth, ignore_thresh, truth_thresh, coord_scale, object_scale,
                         noobject_scale, class_scale);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes,
                           pxh_yolo_workspace_bytes(batch, mask_count, classes, width, height), &ws);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const int blocks = train_blocks(p);
    const YoloTables tb{ assigned_classes, assigned_anchors, assigned_boxes, masks, anchors };
    hipLaunchKernelGGL((yolo_train_kernel<false>), dim3(blocks), dim3(kBlock), 0, s, output, nullptr, delta, truths,
                       truth_counts, p, tb, static_cast<double*>(ws));
    rc = check_launch("yolo_loss");
    if (rc) return rc;
    hipLaunchKernelGGL(yolo_finish_kernel, dim3(1), dim3(kBlock), 0, s, static_cast<const double*>(ws), blocks, stats,
                       cost, 1);
    return check_launch("yolo_finish");
}

}
