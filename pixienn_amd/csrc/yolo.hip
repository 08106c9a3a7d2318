// YOLO head for gfx950: logistic decode, and the training pass (decode + dense delta + cost +
// statistics).
//
// Layout [batch][mask][5 + classes][area].  The training pass is two launches:
//   pass 1  two kinds of workgroup share one grid.  HEAD workgroups give one lane to every slot
//           (image, anchor, cell): the 5 box/objectness rows, the best-truth search, the decision
//           what the slot is supervised with (one int per slot), box/objectness deltas, every
//           statistic and the whole cost (the class rows of the few supervised slots are visited
//           for it).  They are instruction bound.  CLASS workgroups stream the class rows, 94 %
//           of the tensor: logit -> probability -> `out`.  They are bandwidth bound, and the two
//           kinds are interleaved in the grid so that they overlap on every compute unit.
//   pass 2  the dense class delta from the slots' decisions, a write-only stream; its first
//           workgroups also add up the per-workgroup sums of pass 1 in a fixed order.
// Box arithmetic follows the CPU layer (include/YoloLayer.h, src/DarkBox.cpp of the reference).
#include "stream.h"

#include <cfloat>

namespace pxh {
namespace {

constexpr int kMaxAnchors = 32;
constexpr int kMaxMasks = 16;
constexpr int kTruthTile = kBlock;
constexpr int kSums = 12;   // the stats[12] slots; the cost is the sum of slots 8..11

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
    // disjoint boxes (most pairs): 0 / union and the zero-union case both give 0
    if (inter == 0.0f) return 0.0f;
    const float aa = a.w * a.h;
    const float ab = b.w * b.h;
    float uni = aa + ab;
    uni = uni - inter;
    uni = uni > 0.0f ? uni : 0.0f;
    if (uni == 0.0f) return 0.0f;
    return inter / uni;
}

// IoU of a prediction rectangle (pl, pt, pw, ph; not empty) with an unpacked truth: the same
// operations as box_iou, ordered so that a pair that is disjoint along x or along y leaves after
// a handful of instructions.  With lo/hi the rectangles ordered by left edge, the overlap width is
// min(lo.w - (hi.left - lo.left), hi.w) <= lo.w - (hi.left - lo.left): when that bound is not
// positive the intersection is empty whatever the rest says.
__device__ __forceinline__ float rect_iou(float pl, float pt, float pw, float ph, float tl, float tt, float tw,
                                          float th)
{
    const bool p_left = pl < tl;
    const float xlo = p_left ? pl : tl, xlo_w = p_left ? pw : tw;
    const float xhi = p_left ? tl : pl, xhi_w = p_left ? tw : pw;
    const float bx = xlo_w - (xhi - xlo);
    if (!(bx > 0.0f)) return 0.0f;
    const bool p_top = pt < tt;
    const float ylo = p_top ? pt : tt, ylo_h = p_top ? ph : th;
    const float yhi = p_top ? tt : pt, yhi_h = p_top ? th : ph;
    const float by = ylo_h - (yhi - ylo);
    if (!(by > 0.0f)) return 0.0f;
    if ((xlo < 0.0f && xlo + xlo_w < xhi) || (ylo < 0.0f && ylo + ylo_h < yhi)) return 0.0f;
    const float iw = fminf(bx, xhi_w);
    const float ih = fminf(by, yhi_h);
    const float inter = iw * ih;
    if (inter == 0.0f) return 0.0f;
    const float ap = pw * ph;
    const float at = tw * th;
    float uni = ap + at;
    uni = uni - inter;
    uni = uni > 0.0f ? uni : 0.0f;
    if (uni == 0.0f) return 0.0f;
    return inter / uni;
}

// Logistic for the class rows: exp2 and reciprocal in hardware, two multiplies and an add.  The
// argument rounding of v*log2(e) bounds the relative error by |v| * 6e-8 + 2 ulp, well inside
// the 1e-5 the decode is held to, and keeps the class stream bandwidth bound.
__device__ __forceinline__ float sigmoid_fast(float v)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.44269504088896341f));
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

// ---------------------------------------------------------------- training pass
struct YoloParams {
    int batch, mask_count, anchor_count, classes, width, height, area;
    int net_width, net_height, max_truth;
    float ignore_thresh, truth_thresh, coord_scale, object_scale, noobject_scale, class_scale;
    int masks[kMaxMasks];
    float anchors[2 * kMaxAnchors];   // integer pixel sizes held as float
    FastDiv by_tiles;    // workgroups per (image, anchor) in the head sweep
    FastDiv by_masks;
    FastDiv by_width;
    uint32_t blocks;     // workgroups of the head sweep
};

// Tables of the reference's signature (host-built assignment), all device pointers.
struct YoloTables {
    const int* assigned_classes;
    const int* assigned_anchors;
    const float* assigned_boxes;
    const int* masks;
    const float* anchors;
};

// A truth unpacked for the head sweep (32 bytes).  left/top are the rectangle corner DarkBox
// derives (src/DarkBox.cpp:84-118); an empty truth (w <= 0 or h <= 0) gets left = top = +inf so
// that the overlap test below rejects it, as cv::Rect's operator& does.
struct __attribute__((aligned(16))) TruthSlot {
    float left, top, w, h;
    float x, y;
    int cls;
    int target;   // mask_slot * area + cell of the positive this truth claims, or -1
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

// Unpacks one truth and, for the fused pass, finds the positive slot it claims (best anchor over
// ALL anchors against the origin-shifted truth; a positive only if that anchor belongs to this
// head; include/YoloLayer.h:456-482 == src/YoloTargetBuilder.cpp:34-56).
template<bool FUSED>
__device__ __forceinline__ TruthSlot make_truth_slot(const float* __restrict__ g, const YoloParams& p)
{
    TruthSlot s;
    const Box box{ g[0], g[1], g[2], g[3] };
    const bool empty = box.w <= 0.0f || box.h <= 0.0f;
    s.left = empty ? INFINITY : box.x - box.w / 2.0f;
    s.top = empty ? INFINITY : box.y - box.h / 2.0f;
    s.w = box.w; s.h = box.h; s.x = box.x; s.y = box.y;
    s.cls = static_cast<int>(g[4]);
    s.target = -1;
    if constexpr (FUSED) {
        const Box shifted{ 0.0f, 0.0f, box.w, box.h };
        float ba = -FLT_MAX;
        int bi = 0;
        // four anchors at a time: the four IoU chains are independent and overlap in the pipeline
        for (int a0 = 0; a0 < p.anchor_count; a0 += 4) {
            float iou[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int a = min(a0 + u, p.anchor_count - 1);
                const Box cand{ 0.0f, 0.0f, p.anchors[2 * a] / static_cast<float>(p.net_width),
                                p.anchors[2 * a + 1] / static_cast<float>(p.net_height) };
                iou[u] = box_iou(cand, shifted);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (a0 + u < p.anchor_count && iou[u] > ba) { ba = iou[u]; bi = a0 + u; }
        }
        int ms = -1;
        for (int m = 0; m < p.mask_count; ++m)
            if (p.masks[m] == bi) { ms = m; break; }
        if (ms >= 0) {
            int ci = static_cast<int>(box.x * static_cast<float>(p.width));
            int cj = static_cast<int>(box.y * static_cast<float>(p.height));
            ci = max(0, min(ci, p.width - 1));
            cj = max(0, min(cj, p.height - 1));
            // the claimed slot lies on mask `ms`, whose anchor is this truth's best anchor
            s.target = ms * p.area + cj * p.width + ci;
        }
    }
    return s;
}

// probability of class row `c` of the slot at `base`, exactly as the class sweep computes it
template<bool FUSED>
__device__ __forceinline__ float class_prob(const float* in, size_t base, int c, int area)
{
    const float v = in[base + (5 + static_cast<size_t>(c)) * area];
    if constexpr (FUSED) return sigmoid_fast(v);
    else return v;
}

// FUSED: raw logits in, decode written to `out`, positives found from the truths on the device
//        with the CPU layer's rule; statistics as the CPU layer accumulates them.
// !FUSED: `in` is the already decoded head, positives come from the host-built tables;
//        statistics as the reference's device path accumulates them.
// One lane per slot; workgroup `head_block` covers kBlock consecutive cells of one (image, anchor).
struct HeadArgs {
    const float* in;
    float* out;
    float* delta;
    const float* truths;
    const int* truth_counts;
    int* decision;
    double* partial;
};

template<bool FUSED>
__device__ __forceinline__ void head_workgroup(uint32_t head_block, const HeadArgs& a, const YoloParams& p,
                                               const YoloTables& tb, TruthSlot* tile, double* slots)
{
    const float* __restrict__ in = a.in;
    float* __restrict__ out = a.out;
    float* __restrict__ delta = a.delta;
    int* __restrict__ decision = a.decision;
    double* __restrict__ partial = a.partial;
    uint32_t bn, tile_id, b, n;
    p.by_tiles.divmod(head_block, bn, tile_id);
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

    float sx = 0, sy = 0, rw = 0, rh = 0, so = 0;
    if (live) {
        const float v0 = in[base], v1 = in[base + area], v2 = in[base + 2 * static_cast<size_t>(area)],
                    v3 = in[base + 3 * static_cast<size_t>(area)], v4 = in[base + 4 * static_cast<size_t>(area)];
        if constexpr (FUSED) {
            // x, y and objectness feed thresholds and box targets: exact division here
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
    const bool pred_empty = pred.w <= 0.0f || pred.h <= 0.0f;
    const float pl = pred.x - pred.w / 2.0f, pt = pred.y - pred.h / 2.0f;

    // Sweep the image's truths through LDS: best IoU (strict >, first wins) and, in the fused
    // form, the truths that claim this slot as their positive (the last one writes the delta).
    // IoU is never negative, so "first wins from the lowest float" is: start at truth 0 with 0.
    const int count = a.truth_counts[b];
    const float* image_truths = a.truths + static_cast<size_t>(b) * p.max_truth * 5;
    float best = 0.0f;
    int best_k = count > 0 ? 0 : -1;
    int pos_k = -1;
    float st_iou = 0, st_r50 = 0, st_r75 = 0, st_cat = 0, st_obj = 0, st_count = 0;
    const int my_slot = n * area + cell;

    for (int t0 = 0; t0 < count; t0 += kTruthTile) {
        const int t = t0 + threadIdx.x;
        __syncthreads();
        if (t < count) tile[threadIdx.x] = make_truth_slot<FUSED>(image_truths + 5 * static_cast<size_t>(t), p);
        __syncthreads();
        const int tn = min(kTruthTile, count - t0);
        if (live) {
            for (int k = 0; k < tn; ++k) {
                const float4 r = *reinterpret_cast<const float4*>(&tile[k].left);
                const float iou = pred_empty ? 0.0f : rect_iou(pl, pt, pred.w, pred.h, r.x, r.y, r.z, r.w);
                if (iou > best) {
                    best = iou;
                    best_k = t0 + k;
                }
                if constexpr (FUSED) {
                    if (tile[k].target == my_slot) {
                        // every claiming truth is counted (include/YoloLayer.h:480-507); the claimed
                        // slot's anchor is this mask's, so `iou` is the IoU the CPU layer records
                        pos_k = t0 + k;
                        st_cat += fminf(1.0f, class_prob<FUSED>(in, base, tile[k].cls, area));
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

    int pos_cls = -1, pos_anchor = mask_anchor;
    Box pos_box{ 0, 0, 0, 0 };
    if constexpr (FUSED) {
        if (pos_k >= 0) {
            const float* g = image_truths + 5 * static_cast<size_t>(pos_k);
            pos_cls = static_cast<int>(g[4]);
            pos_box = Box{ g[0], g[1], g[2], g[3] };
        }
    } else {
        if (live) {
            const size_t slot = static_cast<size_t>(bn) * area + cell;
            const int acls = tb.assigned_classes[slot];
            if (acls >= 0) {
                pos_cls = acls;
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
                st_cat = fminf(1.0f, class_prob<FUSED>(in, base, acls, area));
            }
        }
    }

    // region decision (include/YoloLayer.h:531-545), then the positive override (480-497)
    float d_obj = 0.0f;
    int cls = -1;            // class the dense class delta is written for, -1: zeros
    BoxDelta bd{ { 0, 0, 0, 0 } };
    float c_box = 0, c_obj = 0, c_noobj = 0, c_cls = 0;
    if (live) {
        const bool have_best = best_k >= 0;
        if (!have_best || best < p.ignore_thresh) d_obj = p.noobject_scale * (0.0f - so);
        if (have_best && best > p.truth_thresh) {
            const float* g = image_truths + 5 * static_cast<size_t>(best_k);
            d_obj = p.object_scale * (1.0f - so);
            cls = static_cast<int>(g[4]);
            bd = box_delta(Box{ g[0], g[1], g[2], g[3] }, sx, sy, rw, rh, i, j, aw, ah, p);
            // deltaYoloClass also feeds the class-probability statistic on this path
            if constexpr (FUSED) st_cat += fminf(1.0f, class_prob<FUSED>(in, base, cls, area));
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
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            delta[base + k * static_cast<size_t>(area)] = bd.v[k];
            c_box += bd.v[k] * bd.v[k];
        }
        delta[base + 4 * static_cast<size_t>(area)] = d_obj;
        if (d_obj >= 0.0f) c_obj = d_obj * d_obj; else c_noobj = d_obj * d_obj;
        decision[static_cast<size_t>(bn) * area + cell] = cls;
        // class deltas are zero except for the supervised slots: their cost is taken here, with
        // the probabilities the class sweep will write
        if (cls >= 0) {
            // 16 independent loads per round trip (rows past the last class re-read it and are
            // masked out); the sum keeps the class order
            constexpr int kRows = 16;
            const float* src = in + base + 5 * static_cast<size_t>(area);
            for (int c0 = 0; c0 < p.classes; c0 += kRows) {
                float v[kRows];
#pragma unroll
                for (int u = 0; u < kRows; ++u) v[u] = src[min(c0 + u, p.classes - 1) * static_cast<size_t>(area)];
#pragma unroll
                for (int u = 0; u < kRows; ++u) {
                    const float prob = FUSED ? sigmoid_fast(v[u]) : v[u];
                    const float t = (c0 + u == cls) ? 1.0f : 0.0f;
                    const float d = p.class_scale * (t - prob);
                    c_cls += (c0 + u < p.classes) ? d * d : 0.0f;
                }
            }
        }
    }

    // Only the objectness sum and the no-object cost exist for every slot; the rest is non-zero
    // only where a slot is supervised, which most workgroups never see.
    const bool any_pos = __syncthreads_or(cls >= 0 || st_count != 0.0f);
    const float sums[12] = { st_iou, st_r50, st_r75, st_cat, st_obj, live ? so : 0.0f, st_count, st_count,
                             c_box, c_obj, c_noobj, c_cls };
    double* dst = partial + head_block;     // [12][blocks]
    const size_t stride = p.blocks;
#pragma unroll
    for (int k = 0; k < 12; ++k) {
        const bool dense = (k == 5 || k == 10);
        if (dense || any_pos) {
            const double total = block_sum(static_cast<double>(sums[k]), slots);
            if (threadIdx.x == 0) dst[k * stride] = total;
        } else if (threadIdx.x == 0) {
            dst[k * stride] = 0.0;
        }
    }
}

// The class rows as a flat index space over [batch*mask][classes][area] (the 5 head rows of every
// anchor are skipped).
struct ClassSpace {
    FastDiv by_area;      // area
    FastDiv by_classes;   // classes
    uint32_t area, entries, elems;
    // flat index e -> (image*mask, class, cell)
    __device__ __forceinline__ void locate(uint32_t e, uint32_t& bn, uint32_t& c, uint32_t& cell) const
    {
        uint32_t rowid;
        by_area.divmod(e, rowid, cell);
        by_classes.divmod(rowid, bn, c);
    }
    __device__ __forceinline__ size_t offset(uint32_t bn, uint32_t c, uint32_t cell) const
    {
        return (static_cast<size_t>(bn) * entries + 5 + c) * area + cell;
    }
};

// ---- pass 1: HEAD workgroups and CLASS (decode) workgroups in one grid ------------------------
struct Pass1Args {
    HeadArgs head;
    ClassSpace space;
    uint32_t head_blocks, class_blocks;   // HEAD workgroups come first in the grid
};

// V = 4 needs area % 4 == 0 (a vector then never leaves its row) and 16-byte aligned tensors.
template<bool FUSED, int V, bool NT>
__global__ __launch_bounds__(kBlock) void yolo_pass1_kernel(Pass1Args a, YoloParams p, YoloTables tb)
{
    __shared__ TruthSlot tile[kTruthTile];
    __shared__ double slots[kBlock / kWave];
    const uint32_t b = blockIdx.x;
    // The long-lived HEAD workgroups are dispatched first, so that the short CLASS workgroups fill the
    // machine as they retire; spreading them through the grid leaves them holding wave slots that
    // the streaming workgroups need.
    if (b < a.head_blocks) {
        head_workgroup<FUSED>(b, a.head, p, tb, tile, slots);
        return;
    }
    if constexpr (FUSED) {
        const uint32_t cb = b - a.head_blocks;
        const uint32_t e = (cb * kBlock + threadIdx.x) * V;
        if (e >= a.space.elems) return;
        uint32_t bn, c, cell;
        a.space.locate(e, bn, c, cell);
        const size_t at = a.space.offset(bn, c, cell);
        const Pack<V> x = ld<V, NT>(a.head.in, at);
        Pack<V> prob;
#pragma unroll
        for (int k = 0; k < V; ++k) prob.v[k] = sigmoid_fast(x.v[k]);
        st<V, NT>(a.head.out, at, prob);
    }
}

// ---- pass 2: dense class delta from the decisions; the first workgroups add up the sums -------
struct Pass2Args {
    const float* prob;     // decoded head (pass 1's `out`, or the caller's decoded input)
    float* delta;
    const int* decision;
    const double* partial;
    float* stats;
    float* cost;
    ClassSpace space;
    uint32_t head_blocks;
    float class_scale;
    int accumulate;
};

// statistic k (k < 12) or the cost (k == 12, slots 8..11) over all HEAD workgroups, fixed order
__device__ __forceinline__ void finish_statistic(int k, const Pass2Args& a, double* slots)
{
    const int first = k < 12 ? k : 8, last = k < 12 ? k : 11;
    double s = 0.0;
    for (int kk = first; kk <= last; ++kk) {
        const double* src = a.partial + static_cast<size_t>(kk) * a.head_blocks;
        for (uint32_t j = threadIdx.x; j < a.head_blocks; j += kBlock) s += src[j];
    }
    const double total = block_sum(s, slots);
    if (threadIdx.x == 0) {
        const float v = static_cast<float>(total);
        if (k < 12) {
            if (a.stats) a.stats[k] = (a.accumulate ? a.stats[k] : 0.0f) + v;
        } else if (a.cost) {
            *a.cost = (a.accumulate ? *a.cost : 0.0f) + v;
        }
    }
}

template<int V, bool NT>
__global__ __launch_bounds__(kBlock) void yolo_pass2_kernel(Pass2Args a)
{
    __shared__ double slots[kBlock / kWave];
    if (blockIdx.x < 13) finish_statistic(blockIdx.x, a, slots);
    const uint32_t e = (blockIdx.x * kBlock + threadIdx.x) * V;
    if (e >= a.space.elems) return;
    uint32_t bn, c, cell;
    a.space.locate(e, bn, c, cell);
    const size_t at = a.space.offset(bn, c, cell);
    const IPack<V> cls = ldi<V, false>(a.decision, static_cast<size_t>(bn) * a.space.area + cell);
    Pack<V> d;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        d.v[k] = 0.0f;
        if (cls.v[k] >= 0) {      // rare: a supervised slot
            const float t = (static_cast<int>(c) == cls.v[k]) ? 1.0f : 0.0f;
            d.v[k] = a.class_scale * (t - a.prob[at + k]);
        }
    }
    st<V, NT>(a.delta, at, d);
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
    p.blocks = static_cast<uint32_t>(batch) * mask_count * tiles;
    return PXH_OK;
}

size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }

// workspace: [12][head workgroups] doubles | one int per slot
struct YoloWorkspace {
    double* partial;
    int* decision;
};

size_t yolo_workspace_bytes(int batch, int mask_count, int width, int height)
{
    const size_t area = static_cast<size_t>(width) * height;
    const size_t tiles = (area + kBlock - 1) / kBlock;
    return align256(static_cast<size_t>(batch) * mask_count * tiles * kSums * sizeof(double)) +
           align256(static_cast<size_t>(batch) * mask_count * area * sizeof(int));
}

YoloWorkspace carve(void* ws, const YoloParams& p)
{
    YoloWorkspace w;
    char* c = static_cast<char*>(ws);
    w.partial = reinterpret_cast<double*>(c);
    c += align256(static_cast<size_t>(p.blocks) * kSums * sizeof(double));
    w.decision = reinterpret_cast<int*>(c);
    return w;
}

template<bool FUSED>
int run_training_pass(const char* who, const float* in, float* out, float* delta, const float* truths,
                      const int* truth_counts, const YoloParams& p, const YoloTables& tb, float* stats, float* cost,
                      int accumulate, void* ws, hipStream_t s)
{
    const YoloWorkspace w = carve(ws, p);
    ClassSpace space{ FastDiv(p.area), FastDiv(p.classes), static_cast<uint32_t>(p.area),
                      static_cast<uint32_t>(p.classes + 5),
                      static_cast<uint32_t>(static_cast<size_t>(p.batch) * p.mask_count * p.classes * p.area) };
    const bool vec = p.area % 4 == 0 && aligned16(in) && aligned16(out) && aligned16(delta);
    const uint32_t per_block = kBlock * (vec ? 4 : 1);
    const uint32_t class_blocks = (space.elems + per_block - 1) / per_block;

    Pass1Args a1{};
    a1.head = HeadArgs{ in, out, delta, truths, truth_counts, w.decision, w.partial };
    a1.space = space;
    a1.head_blocks = p.blocks;
    a1.class_blocks = FUSED ? class_blocks : 0;
    const uint32_t total1 = a1.head_blocks + a1.class_blocks;
    const bool nt1 = static_cast<size_t>(space.elems) * 8 >= kStreamingBytes;
    if (vec && nt1) hipLaunchKernelGGL((yolo_pass1_kernel<FUSED, 4, true>), dim3(total1), dim3(kBlock), 0, s, a1, p, tb);
    else if (vec) hipLaunchKernelGGL((yolo_pass1_kernel<FUSED, 4, false>), dim3(total1), dim3(kBlock), 0, s, a1, p, tb);
    else hipLaunchKernelGGL((yolo_pass1_kernel<FUSED, 1, false>), dim3(total1), dim3(kBlock), 0, s, a1, p, tb);
    int rc = check_launch(who);
    if (rc) return rc;

    Pass2Args a2{};
    a2.prob = FUSED ? out : in;
    a2.delta = delta;
    a2.decision = w.decision;
    a2.partial = w.partial;
    a2.stats = stats;
    a2.cost = cost;
    a2.space = space;
    a2.head_blocks = p.blocks;
    a2.class_scale = p.class_scale;
    a2.accumulate = accumulate;
    const uint32_t total2 = class_blocks < 13 ? 13 : class_blocks;
    const bool nt2 = static_cast<size_t>(space.elems) * 4 >= kStreamingBytes;
    if (vec && nt2) hipLaunchKernelGGL((yolo_pass2_kernel<4, true>), dim3(total2), dim3(kBlock), 0, s, a2);
    else if (vec) hipLaunchKernelGGL((yolo_pass2_kernel<4, false>), dim3(total2), dim3(kBlock), 0, s, a2);
    else hipLaunchKernelGGL((yolo_pass2_kernel<1, false>), dim3(total2), dim3(kBlock), 0, s, a2);
    return check_launch(who);
}

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

size_t pxh_yolo_workspace_bytes(int batch, int mask_count, int classes, int width, int height, int max_truth)
{
    (void) classes;
    (void) max_truth;
    if (batch <= 0 || mask_count <= 0 || width <= 0 || height <= 0) return 0;
    return yolo_workspace_bytes(batch, mask_count, width, height);
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
                           yolo_workspace_bytes(batch, mask_count, width, height), &ws);
    if (rc) return rc;
    return run_training_pass<true>("pxh_yolo_forward_train", input, output, delta, truths, truth_counts, p,
                                   YoloTables{}, stats, cost, 0, ws, as_stream(stream));
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
                           yolo_workspace_bytes(batch, mask_count, width, height), &ws);
    if (rc) return rc;
    const YoloTables tb{ assigned_classes, assigned_anchors, assigned_boxes, masks, anchors };
    return run_training_pass<false>("pxh_yolo_loss", output, nullptr, delta, truths, truth_counts, p, tb, stats,
                                    cost, 1, ws, as_stream(stream));
}

}
