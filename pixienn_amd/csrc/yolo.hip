// YOLO head for gfx950: logistic decode, and the training pass (decode + dense delta + cost +
// statistics).
//
// Layout [batch][mask][5 + classes][area].  The work of the training pass has two parts:
//   head   one lane per slot (image, anchor, cell): the 5 box/objectness rows, the best-truth
//          search against the image's truths staged in LDS, the decision what the slot is
//          supervised with (one int per slot), box/objectness deltas, every statistic and the
//          whole cost (the class rows of the few supervised slots are visited for it).
//          Instruction and latency bound: ~1000 vector instructions per wave.
//   class  the class rows, 94 % of the tensor: logit -> probability -> `out`, and the dense class
//          delta.  Bandwidth bound, 12 bytes per element.
// Both run in ONE grid, persistent head workgroups beside the class stream.  Two forms of the pass,
// picked by the size of the head (run_training_pass): in ONE launch for small heads, whose time is a
// head tile's chain of dependent steps -- the head tiles write every delta of their cells, a slot's
// truth sweep is spread over two lanes, and the workgroup that finishes last adds up the sums; in TWO
// launches for large heads, whose time is the class stream's -- the stream also writes the zero
// class deltas, and a small second kernel writes the class deltas of the few supervised slots and
// adds up the sums.
// pxh_yolo_forward_train starts from raw logits and assigns the positives on the device;
// pxh_yolo_loss (the reference's argument list) starts from a decoded head and host-assigned
// positives.  pxh_yolo_detections is the inference-side compaction.
// Box arithmetic follows the CPU layer (include/YoloLayer.h, src/DarkBox.cpp of the reference).
#include "stream.h"
#include "pixienn_hip_test.h"

#include <atomic>
#include <cfloat>
#include <mutex>
#include <vector>

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

// Overlap area of a prediction rectangle (pl, pt, pw, ph; not empty) with an unpacked truth: the
// operations of box_intersection without its branches, so that several pairs can be in flight
// in one lane.  With lo/hi the rectangles ordered by left edge, the overlap width is
// min(lo.w - (hi.left - lo.left), hi.w); an empty truth carries left = +inf and drops out here.
__device__ __forceinline__ float rect_overlap(float pl, float pt, float pw, float ph, float tl, float tt, float tw,
                                              float th)
{
    const bool p_left = pl < tl;
    const float xlo = p_left ? pl : tl, xlo_w = p_left ? pw : tw;
    const float xhi = p_left ? tl : pl, xhi_w = p_left ? tw : pw;
    const float bx = xlo_w - (xhi - xlo);
    const bool p_top = pt < tt;
    const float ylo = p_top ? pt : tt, ylo_h = p_top ? ph : th;
    const float yhi = p_top ? tt : pt, yhi_h = p_top ? th : ph;
    const float by = ylo_h - (yhi - ylo);
    // bitwise on purpose: no short-circuit branches, the lanes of a wave rarely agree
    const bool meet = (bx > 0.0f) & (by > 0.0f) & !((xlo < 0.0f) & (xlo + xlo_w < xhi)) &
                      !((ylo < 0.0f) & (ylo + ylo_h < yhi));
    const float iw = fminf(bx, xhi_w);
    const float ih = fminf(by, yhi_h);
    return meet ? iw * ih : 0.0f;
}

// inter / union as box_iou forms it; 0 when either is 0.  No branches.
__device__ __forceinline__ float overlap_ratio(float inter, float pw, float ph, float tw, float th)
{
    const float ap = pw * ph;
    const float at = tw * th;
    float uni = ap + at;
    uni = uni - inter;
    const bool some = (uni > 0.0f) & (inter > 0.0f);
    const float q = inter / (some ? uni : 1.0f);
    return some ? q : 0.0f;
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
    float anchors_rel[2 * kMaxAnchors];   // anchors[2a] / net_width, anchors[2a+1] / net_height (fp32 division)
    FastDiv by_tiles;    // head tiles per (image, anchor)
    FastDiv by_masks;
    FastDiv by_width;
    FastDiv by_anchors;
    FastDiv by_area;
    uint32_t blocks;     // head tiles in all
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

// probability of class row `c` of the slot at `base`, exactly as the class sweep computes it
template<bool FUSED>
__device__ __forceinline__ float class_prob(const float* in, size_t base, int c, int area, int classes)
{
    if (c < 0 || c >= classes) return 0.0f;      // a label outside the class range reads nothing
    const float v = in[base + (5 + static_cast<size_t>(c)) * area];
    if constexpr (FUSED) return sigmoid_fast(v);
    else return v;
}

// Sum of 64 lanes, pairwise (butterfly): at most 6 roundings on any path.
__device__ __forceinline__ float wave_sum_pairwise(float v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

constexpr int kWaves = kBlock / kWave;

// ==========================================================================================
// The training pass in ONE launch: persistent head workgroups that own every delta of their
// cells, a class stream that only decodes, the final sums inside the same launch.  The form for
// heads up to a hundred megabytes or so, whose time is one head tile's chain of dependent steps:
// there it saves the second launch and shortens the chain (several lanes per slot).
// ==========================================================================================
namespace one_launch {

// Unpacks one truth; which slot it claims is found afterwards (claim_targets).
__device__ __forceinline__ TruthSlot make_truth_slot(const float* __restrict__ g)
{
    TruthSlot s;
    const Box box{ g[0], g[1], g[2], g[3] };
    const bool empty = box.w <= 0.0f || box.h <= 0.0f;
    s.left = empty ? INFINITY : box.x - box.w / 2.0f;
    s.top = empty ? INFINITY : box.y - box.h / 2.0f;
    s.w = box.w; s.h = box.h; s.x = box.x; s.y = box.y;
    s.cls = static_cast<int>(g[4]);
    s.target = -1;
    return s;
}

// IoU of a truth of size (w, h) with an anchor of size (cw, ch), both centred on the origin, where
// DarkBox's rectangle intersection reduces to min(w) * min(h) exactly: ordered by left edge the wider
// box comes first, its overlap bound W - (W/2 - n/2) is never below the narrower width n, and the
// negative-left test (-W/2 + W < -n/2) is false.  The ratio is then formed as box_iou forms it.
__device__ __forceinline__ float anchor_iou(float w, float h, float cw, float ch)
{
    const bool none = (w <= 0.0f) | (h <= 0.0f) | (cw <= 0.0f) | (ch <= 0.0f);
    const float inter = none ? 0.0f : fminf(cw, w) * fminf(ch, h);
    const float aa = cw * ch;
    const float ab = w * h;
    float uni = aa + ab;
    uni = uni - inter;
    const bool some = (uni > 0.0f) & (inter > 0.0f);
    const float q = inter / (some ? uni : 1.0f);
    return some ? q : 0.0f;
}

// The cell a truth's centre falls into (include/YoloLayer.h:470-476): whichever anchor claims a slot
// for the truth, it is a slot of this cell.
__device__ __forceinline__ int truth_cell(float x, float y, const YoloParams& p)
{
    int ci = static_cast<int>(x * static_cast<float>(p.width));
    int cj = static_cast<int>(y * static_cast<float>(p.height));
    ci = max(0, min(ci, p.width - 1));
    cj = max(0, min(cj, p.height - 1));
    return cj * p.width + ci;
}

// The positive slot staged truth `t` claims, from its IoU with every anchor (row[a]): the best anchor
// over ALL anchors (strict >, the first wins); a positive only if that anchor belongs to this head, at
// the cell the truth's centre falls into (include/YoloLayer.h:456-482 ==
// src/YoloTargetBuilder.cpp:34-56).
__device__ __forceinline__ void pick_target(TruthSlot* tile, int t, const float* row, const YoloParams& p)
{
    float ba = -FLT_MAX;
    int bi = 0;
    for (int a = 0; a < p.anchor_count; ++a) {
        const float iou = row[a];
        const bool better = iou > ba;
        ba = better ? iou : ba;
        bi = better ? a : bi;
    }
    int ms = -1;
    for (int m = 0; m < p.mask_count; ++m)
        if (p.masks[m] == bi) { ms = m; break; }
    // the claimed slot lies on mask `ms`, whose anchor is this truth's best anchor
    if (ms >= 0) tile[t].target = ms * p.area + truth_cell(tile[t].x, tile[t].y, p);
}

// The same for all `tn` staged truths, however many: one (truth, anchor) pair per lane, so that the
// divisions of a truth run side by side instead of one after the other; then one lane per truth
// picks the best.  Called by the whole workgroup, between barriers of its own.
__device__ __forceinline__ void claim_targets(TruthSlot* tile, int tn, float* pair_iou, const YoloParams& p)
{
    const int per = kBlock / p.anchor_count;       // truths per pass (anchor_count <= kMaxAnchors <= kBlock)
    uint32_t tt, aa;
    p.by_anchors.divmod(threadIdx.x, tt, aa);
    for (int c0 = 0; c0 < tn; c0 += per) {
        const int t = c0 + static_cast<int>(tt);
        if (static_cast<int>(tt) < per && t < tn)
            pair_iou[threadIdx.x] = anchor_iou(tile[t].w, tile[t].h, p.anchors_rel[2 * aa], p.anchors_rel[2 * aa + 1]);
        __syncthreads();
        const int mine = c0 + static_cast<int>(threadIdx.x);
        if (static_cast<int>(threadIdx.x) < per && mine < tn) pick_target(tile, mine, pair_iou + threadIdx.x * p.anchor_count, p);
        __syncthreads();
    }
}

// FUSED: raw logits in, decode written to `out`, positives found from the truths on the device
//        with the CPU layer's rule; statistics as the CPU layer accumulates them.
// !FUSED: `in` is the already decoded head, positives come from the host-built tables;
//        statistics as the reference's device path accumulates them.
struct HeadArgs {
    const float* in;
    float* out;
    float* delta;
    const float* truths;
    const int* truth_counts;
    int wide_delta;      // delta is 16-byte aligned and area % 4 == 0: the class rows are cleared 4 cells at a time
};

// One head tile: kBlock / L consecutive cells of one (image, anchor), L lanes per slot (image, anchor,
// cell).  Every lane of a slot decodes the slot's box and objectness; the image's truths, staged in
// LDS, are dealt round-robin to the L lanes for the overlap sweep and the results are combined with
// the rules of the sequential sweep (best IoU: strict >, the first truth wins; positive: the last
// claiming truth wins).  The tile writes the box and objectness deltas and ALL class deltas of its
// cells (zeros, except at the few supervised slots) and returns its share of the 12 sums.
// Small heads (19 x 19 at any batch) have far fewer slots than the machine has lanes and are bound by
// the length of this instruction stream: L > 1 shortens the sweep and gives the machine L times as
// many waves to run side by side.
// Returns, in threads 0..kSums-1, the tile's sum of statistic threadIdx.x.
template<bool FUSED, int L, bool NT>
__device__ __forceinline__ double head_tile(const uint32_t head_block, const HeadArgs& a, const YoloParams& p,
                                            const YoloTables& tb, TruthSlot* tile, float* pair_iou,
                                            double (*wave_sums)[kWaves])
{
    static_assert(L == 1 || L == 2 || L == 4, "lanes per slot");
    constexpr int kCells = kBlock / L;
    const float* __restrict__ in = a.in;
    float* __restrict__ out = a.out;
    float* __restrict__ delta = a.delta;
    uint32_t bn, tile_id, b, n;
    p.by_tiles.divmod(head_block, bn, tile_id);
    p.by_masks.divmod(bn, b, n);
    const int sub = threadIdx.x & (L - 1);
    const int cell = tile_id * kCells + threadIdx.x / L;
    const bool live = cell < p.area;
    const bool lead = live && sub == 0;        // the lane that stands for its slot in stores and sums
    const int area = p.area;
    const int entries = p.classes + 5;
    const size_t base = (static_cast<size_t>(bn) * entries) * area + (live ? cell : 0);

    // Asked for first, used last: the truth count, this lane's truth of the image and, for the search of
    // each truth's best anchor, the (truth, anchor) pair this lane evaluates.  None of the addresses
    // depends on another load, so all of it travels together with the head rows below.
    // a count beyond the table's rows must not read past them
    const int count = min(a.truth_counts[b], p.max_truth);
    const float* image_truths = a.truths + static_cast<size_t>(b) * p.max_truth * 5;
    float mine[5] = { 0, 0, 0, 0, 0 };
    if (static_cast<int>(threadIdx.x) < p.max_truth) {
#pragma unroll
        for (int k = 0; k < 5; ++k) mine[k] = image_truths[5 * static_cast<size_t>(threadIdx.x) + k];
    }
    uint32_t pair_truth = 0, pair_anchor = 0;
    float pair_w = 0, pair_h = 0, pair_cw = 0, pair_ch = 0;
    if constexpr (FUSED) {
        p.by_anchors.divmod(threadIdx.x, pair_truth, pair_anchor);
        if (static_cast<int>(pair_truth) < p.max_truth) {
            pair_w = image_truths[5 * static_cast<size_t>(pair_truth) + 2];
            pair_h = image_truths[5 * static_cast<size_t>(pair_truth) + 3];
        }
        pair_cw = p.anchors_rel[2 * pair_anchor];
        pair_ch = p.anchors_rel[2 * pair_anchor + 1];
    }

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
    // the host-built table says whether something supervises this slot: asked for with the head rows
    // (it is needed after the sweep, where it would be a trip to memory of its own)
    int table_cls = -1;
    if constexpr (!FUSED) {
        if (live) table_cls = tb.assigned_classes[static_cast<size_t>(bn) * area + cell];
    }
    if (live) {
        const float v0 = in[base], v1 = in[base + area], v2 = in[base + 2 * static_cast<size_t>(area)],
                    v3 = in[base + 3 * static_cast<size_t>(area)], v4 = in[base + 4 * static_cast<size_t>(area)];
        if constexpr (FUSED) {
            // x, y and objectness feed thresholds and box targets: exact division here
            sx = 1.0f / (1.0f + expf(-v0));
            sy = 1.0f / (1.0f + expf(-v1));
            so = 1.0f / (1.0f + expf(-v4));
            if (lead) {
                out[base] = sx;
                out[base + area] = sy;
                out[base + 2 * static_cast<size_t>(area)] = v2;
                out[base + 3 * static_cast<size_t>(area)] = v3;
                out[base + 4 * static_cast<size_t>(area)] = so;
            }
        } else {
            sx = v0; sy = v1; so = v4;
        }
        rw = v2; rh = v3;
    }
    // The class deltas of the tile are zero except at the few slots something supervises: cleared now
    // (behind the loads above, which the memory pipeline serves in the order they were asked for), so
    // that the stores are on their way while the truths are swept.  Every wave clears the rows of its
    // own cells; where a slot turns out to be supervised, the same wave writes its class deltas later,
    // after these stores have been acknowledged.
    {
        constexpr int kWaveCells = kWave / L;
        const int lane_ = threadIdx.x & (kWave - 1);
        const int wave_cell0 = tile_id * kCells + (threadIdx.x / kWave) * kWaveCells;
        float* rows = delta + (static_cast<size_t>(bn) * entries + 5) * area;
        if (a.wide_delta && kWaveCells >= 4) {
            constexpr int kVec = kWaveCells >= 4 ? kWaveCells / 4 : 1;      // vectors per row and wave
            Pack<4> zero;
#pragma unroll
            for (int k = 0; k < 4; ++k) zero.v[k] = 0.0f;
            for (int v = lane_; v < p.classes * kVec; v += kWave) {
                const int r = v / kVec, c = wave_cell0 + (v % kVec) * 4;
                if (c < area) st<4, NT>(rows, static_cast<size_t>(r) * area + c, zero);
            }
        } else {
            for (int v = lane_; v < p.classes * kWaveCells; v += kWave) {
                const int r = v / kWaveCells, c = wave_cell0 + v % kWaveCells;
                if (c < area) rows[static_cast<size_t>(r) * area + c] = 0.0f;
            }
        }
    }

    const Box pred = decode_box(sx, sy, rw, rh, i, j, aw, ah, p);
    const bool pred_empty = pred.w <= 0.0f || pred.h <= 0.0f;
    // an empty prediction overlaps nothing: park it where every overlap test fails
    const float pl = pred_empty ? INFINITY : pred.x - pred.w / 2.0f, pt = pred.y - pred.h / 2.0f;

    // Sweep the image's truths through LDS: best IoU (strict >, first wins) and, in the fused
    // form, the truths that claim this slot as their positive (the last one writes the delta).
    // IoU is never negative, so "first wins from the lowest float" is: start at truth 0 with 0.
    float best = 0.0f;
    int best_k = count > 0 ? 0 : -1;
    int pos_cls = -1, pos_anchor = mask_anchor, pos_t = -1;
    Box pos_box{ 0, 0, 0, 0 };
    float st_iou = 0, st_r50 = 0, st_r75 = 0, st_cat = 0, st_obj = 0, st_count = 0;
    const int my_slot = live ? static_cast<int>(n) * area + cell : -2;
    // truths per step and lane: their overlap tests are independent and interleave
    constexpr int kUnroll = L == 1 ? 4 : 2;

    for (int t0 = 0; t0 < count; t0 += kTruthTile) {
        const int t = t0 + threadIdx.x;
        const int tn = min(kTruthTile, count - t0);
        __syncthreads();       // the previous tile (or the previous head tile of this workgroup) is done with
        // the first tile of truths comes from the registers filled at the top
        const bool quick = FUSED && t0 == 0 && tn <= kBlock / p.anchor_count;
        if (t0 == 0) {
            if (t < count) tile[threadIdx.x] = make_truth_slot(mine);
            if (quick && static_cast<int>(pair_truth) < tn)
                pair_iou[threadIdx.x] = anchor_iou(pair_w, pair_h, pair_cw, pair_ch);
        } else if (t < count) {
            tile[threadIdx.x] = make_truth_slot(image_truths + 5 * static_cast<size_t>(t));
        }
        __syncthreads();
        if constexpr (FUSED) {
            if (quick) {
                if (static_cast<int>(threadIdx.x) < tn) pick_target(tile, threadIdx.x, pair_iou + threadIdx.x * p.anchor_count, p);
                __syncthreads();
            } else {
                claim_targets(tile, tn, pair_iou, p);
            }
        }
        // The lanes of a slot take the truths in turn (lane `sub`: sub, sub + L, ...), kUnroll per step;
        // inside a lane the ordered part (best so far, claims) follows in truth order.  Steps past the
        // last truth re-read it with an empty overlap and no target.
        for (int k0 = 0; k0 < tn; k0 += kUnroll * L) {
            float inter[kUnroll], tw[kUnroll], th[kUnroll], iou[kUnroll];
            int target[kUnroll], at[kUnroll];
            bool touch = false, claimed = false;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int idx = k0 + u * L + sub;
                const bool real = idx < tn;
                at[u] = real ? idx : tn - 1;
                const float4 r = *reinterpret_cast<const float4*>(&tile[at[u]].left);
                target[u] = real ? tile[at[u]].target : -1;
                tw[u] = r.z; th[u] = r.w;
                const float ov = rect_overlap(pl, pt, pred.w, pred.h, r.x, r.y, r.z, r.w);
                inter[u] = real ? ov : 0.0f;
                touch = touch | (inter[u] > 0.0f);
                claimed = claimed | (target[u] == my_slot);
            }
            // most steps touch nothing in the whole wave: no divisions then
            if (__ballot(touch)) {
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) iou[u] = overlap_ratio(inter[u], pred.w, pred.h, tw[u], th[u]);
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const bool better = iou[u] > best;
                    best = better ? iou[u] : best;
                    best_k = better ? t0 + at[u] : best_k;
                }
            } else {
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) iou[u] = 0.0f;
            }
            if constexpr (FUSED) {
                if (__ballot(claimed)) {
#pragma unroll
                    for (int u = 0; u < kUnroll; ++u) {
                        if (target[u] == my_slot) {
                            // every claiming truth is counted (include/YoloLayer.h:480-507); the claimed
                            // slot's anchor is this mask's, so iou[u] is the IoU the CPU layer records
                            const TruthSlot& ts = tile[at[u]];
                            pos_t = t0 + at[u];
                            pos_cls = ts.cls;
                            pos_box = Box{ ts.x, ts.y, ts.w, ts.h };
                            st_cat += fminf(1.0f, class_prob<FUSED>(in, base, ts.cls, area, p.classes));
                            st_iou += iou[u];
                            if (iou[u] > .5f) st_r50 += 1.0f;
                            if (iou[u] > .75f) st_r75 += 1.0f;
                            st_obj += so;
                            st_count += 1.0f;
                        }
                    }
                }
            }
        }
    }

    // What the L lanes of a slot found, combined as the sequential sweep would have it: the larger
    // IoU, on a tie the earlier truth; the positive of the latest claiming truth; the statistics of
    // all claiming truths.  Afterwards every lane of the slot holds the slot's values.
    if constexpr (L > 1) {
#pragma unroll
        for (int off = 1; off < L; off <<= 1) {
            const float o_best = __shfl_xor(best, off, kWave);
            const int o_k = __shfl_xor(best_k, off, kWave);
            const bool take = (o_best > best) | ((o_best == best) & (o_k < best_k));
            best = take ? o_best : best;
            best_k = take ? o_k : best_k;
        }
        if constexpr (FUSED) {
            if (__ballot(pos_t >= 0)) {
#pragma unroll
                for (int off = 1; off < L; off <<= 1) {
                    const int o_t = __shfl_xor(pos_t, off, kWave);
                    const int o_cls = __shfl_xor(pos_cls, off, kWave);
                    const float ox = __shfl_xor(pos_box.x, off, kWave), oy = __shfl_xor(pos_box.y, off, kWave);
                    const float ow = __shfl_xor(pos_box.w, off, kWave), oh = __shfl_xor(pos_box.h, off, kWave);
                    const bool take = o_t > pos_t;
                    pos_t = take ? o_t : pos_t;
                    pos_cls = take ? o_cls : pos_cls;
                    pos_box = take ? Box{ ox, oy, ow, oh } : pos_box;
                    st_cat += __shfl_xor(st_cat, off, kWave);
                    st_iou += __shfl_xor(st_iou, off, kWave);
                    st_r50 += __shfl_xor(st_r50, off, kWave);
                    st_r75 += __shfl_xor(st_r75, off, kWave);
                    st_obj += __shfl_xor(st_obj, off, kWave);
                    st_count += __shfl_xor(st_count, off, kWave);
                }
            }
        }
    }

    if constexpr (!FUSED) {
        if (live) {
            const size_t slot = static_cast<size_t>(bn) * area + cell;
            const int acls = table_cls;
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
                st_cat = fminf(1.0f, class_prob<FUSED>(in, base, acls, area, p.classes));
            }
        }
    }

    // region decision (include/YoloLayer.h:531-545), then the positive override (480-497)
    float d_obj = 0.0f;
    int cls = -1;            // class the dense class delta is written for, -1: zeros
    BoxDelta bd{ { 0, 0, 0, 0 } };
    float c_box = 0, c_obj = 0, c_noobj = 0;
    if (live) {
        const bool have_best = best_k >= 0;
        if (!have_best || best < p.ignore_thresh) d_obj = p.noobject_scale * (0.0f - so);
        if (have_best && best > p.truth_thresh) {
            const float* g = image_truths + 5 * static_cast<size_t>(best_k);
            d_obj = p.object_scale * (1.0f - so);
            cls = static_cast<int>(g[4]);
            bd = box_delta(Box{ g[0], g[1], g[2], g[3] }, sx, sy, rw, rh, i, j, aw, ah, p);
            // deltaYoloClass also feeds the class-probability statistic on this path
            if constexpr (FUSED) st_cat += fminf(1.0f, class_prob<FUSED>(in, base, cls, area, p.classes));
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
        for (int k = 0; k < 4; ++k) c_box += bd.v[k] * bd.v[k];
        if (d_obj >= 0.0f) c_obj = d_obj * d_obj; else c_noobj = d_obj * d_obj;
        if (lead) {
#pragma unroll
            for (int k = 0; k < 4; ++k) delta[base + k * static_cast<size_t>(area)] = bd.v[k];
            delta[base + 4 * static_cast<size_t>(area)] = d_obj;
        }
    }

    // Workgroup sums.  The objectness sum and the no-object cost exist for every slot: pairwise
    // over the wave.  Everything else is non-zero only at supervised slots, which most waves never
    // see: their lead lanes are visited one by one, in lane order.  The class deltas of such a slot
    // are written here, by the whole wave together, one class row per lane, with the probabilities
    // the class stream writes (the same function of the same logits), and their cost is taken.
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const float dense_obj = wave_sum_pairwise(lead ? so : 0.0f);
    const float dense_noobj = wave_sum_pairwise(lead ? c_noobj : 0.0f);
    const float sparse[9] = { st_iou, st_r50, st_r75, st_cat, st_obj, st_count, st_count, c_box, c_obj };
    constexpr int slot_of[9] = { 0, 1, 2, 3, 4, 6, 7, 8, 9 };
    double acc[9] = { 0, 0, 0, 0, 0, 0, 0, 0, 0 };
    double class_cost = 0.0;
    unsigned long long todo = __ballot(lead && (cls >= 0 || st_count != 0.0f));
    unsigned long long supervised = __ballot(lead && cls >= 0);
    while (todo) {
        const int src_lane = __builtin_ctzll(todo);
        todo &= todo - 1;
#pragma unroll
        for (int k = 0; k < 9; ++k)
            acc[k] += static_cast<double>(__shfl(sparse[k], src_lane, kWave));
    }
    // this wave cleared these class rows at the top of the tile: those stores are through first
    if (supervised) __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    // kTogether slots at a time, so that their class rows are fetched in one trip
    constexpr int kTogether = 4;
    while (supervised) {
        int s_cls[kTogether];
        size_t first[kTogether];
#pragma unroll
        for (int q = 0; q < kTogether; ++q) {
            const bool some = supervised != 0;
            const int src_lane = some ? __builtin_ctzll(supervised) : 0;
            supervised &= supervised - 1;      // 0 stays 0
            s_cls[q] = some ? __shfl(cls, src_lane, kWave) : -1;
            first[q] = (static_cast<size_t>(bn) * entries + 5) * area + __shfl(cell, src_lane, kWave);
        }
        float sq[kTogether];
#pragma unroll
        for (int q = 0; q < kTogether; ++q) sq[q] = 0.0f;
        for (int c = lane; c < p.classes; c += kWave) {
            float v[kTogether];
#pragma unroll
            for (int q = 0; q < kTogether; ++q) v[q] = s_cls[q] >= 0 ? in[first[q] + static_cast<size_t>(c) * area] : 0.0f;
#pragma unroll
            for (int q = 0; q < kTogether; ++q) {
                if (s_cls[q] >= 0) {
                    const float prob = FUSED ? sigmoid_fast(v[q]) : v[q];
                    const float t = (c == s_cls[q]) ? 1.0f : 0.0f;
                    const float d = p.class_scale * (t - prob);
                    delta[first[q] + static_cast<size_t>(c) * area] = d;
                    sq[q] += d * d;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < kTogether; ++q)
            if (s_cls[q] >= 0) class_cost += static_cast<double>(wave_sum_pairwise(sq[q]));
    }
    if (lane == 0) {
#pragma unroll
        for (int k = 0; k < 9; ++k) wave_sums[slot_of[k]][wave] = acc[k];
        wave_sums[5][wave] = static_cast<double>(dense_obj);
        wave_sums[10][wave] = static_cast<double>(dense_noobj);
        wave_sums[11][wave] = class_cost;
    }
    __syncthreads();
    double total = 0.0;
    if (threadIdx.x < kSums) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total += wave_sums[threadIdx.x][w];
    }
    return total;
}

// The class rows of one (image, anchor) are one contiguous run of classes * area floats (row after
// row).  The class stream walks every run in 128-bit vectors at 16-byte aligned addresses, whatever
// the area: a run that starts `mis` floats past such an address gets one vector slot more, and the
// slots at its two ends, which reach outside the run, are worked element by element.
struct ClassRuns {
    FastDiv by_slots;        // vector slots per run: (run_len + 3 + 3) / 4, enough for any start
    uint32_t run_len;        // classes * area
    uint32_t run_stride;     // (classes + 5) * area, from one run to the next
    uint32_t first;          // 5 * area, the start of the first run
    uint32_t total_slots;    // runs * slots per run
    uint32_t elems;          // runs * run_len (for the element-wise form)
    FastDiv by_run_len;
};

constexpr int kClassVectors = 4;      // vectors a lane of the class stream has in flight

// Block `block` of the class stream: kClassVectors vector slots per lane, a workgroup-wide stride
// apart, logit -> probability.
template<bool NT>
__device__ __forceinline__ void class_stream_block(const float* __restrict__ in, float* __restrict__ out,
                                                   const ClassRuns& r, uint32_t block)
{
    size_t start[kClassVectors];
    int lo[kClassVectors];
    bool live[kClassVectors], whole[kClassVectors];
    Pack<4> x[kClassVectors];
#pragma unroll
    for (int u = 0; u < kClassVectors; ++u) {
        const uint32_t g = (block * kClassVectors + u) * kBlock + threadIdx.x;
        live[u] = g < r.total_slots;
        uint32_t run, slot;
        r.by_slots.divmod(live[u] ? g : 0u, run, slot);
        start[u] = static_cast<size_t>(run) * r.run_stride + r.first;
        lo[u] = static_cast<int>(slot * 4) - static_cast<int>(start[u] & 3);     // first element of the slot, in the run
        whole[u] = live[u] && lo[u] >= 0 && lo[u] + 3 < static_cast<int>(r.run_len);
        if (whole[u]) x[u] = ld<4, NT>(in, start[u] + lo[u]);
    }
#pragma unroll
    for (int u = 0; u < kClassVectors; ++u) {
        if (whole[u]) {
            Pack<4> prob;
#pragma unroll
            for (int k = 0; k < 4; ++k) prob.v[k] = sigmoid_fast(x[u].v[k]);
            st<4, NT>(out, start[u] + lo[u], prob);
        } else if (live[u]) {
            for (int k = 0; k < 4; ++k) {
                const int e = lo[u] + k;
                if (e >= 0 && e < static_cast<int>(r.run_len)) out[start[u] + e] = sigmoid_fast(in[start[u] + e]);
            }
        }
    }
}

// ---- adding up the head workers' sums inside the same launch -----------------------------------
// Every head worker leaves its 12 sums in memory and "arrives" at a counter; the worker that arrives
// last adds up what all of them left, in a fixed order (worker by worker), so the totals do not depend
// on which worker that was.  Nothing waits: a worker that is not last simply ends.  Two levels
// (groups of kGroup workers, then the groups) keep both the number of values one workgroup reads
// and the number of arrivals at one counter small: device-scope atomic operations on one address
// take some 15 ns each, one after the other.
//
// A counter is a 64-bit word that is 0 whenever no launch is using it: arrivals add 1, the last one
// puts the 0 back.  The counters live in device memory of the library's own (g_arrival_counters below,
// zero when the code object is loaded), not in the workspace, whose contents nobody vouches for: a set
// of counters per workspace address the library has seen, so that launches which may overlap -- they
// have workspaces of their own -- never share one.  Each counter has a cache line of its own, so
// that the groups do not queue behind each other at one memory channel.
constexpr int kGroup = 256;
constexpr uint32_t kMaxWorkers = 2048;
constexpr uint32_t kMaxGroups = kMaxWorkers / kGroup;
constexpr int kCounterStride = 256 / sizeof(unsigned long long);      // words between two counters

constexpr int kCountersPerSet = 1 + kMaxGroups;
constexpr int kCounterSets = 256;
__device__ __align__(256) unsigned long long g_arrival_counters[kCounterSets * kCountersPerSet * kCounterStride];

// True for the last of `members` arrivals.
__device__ __forceinline__ bool arrive(unsigned long long* word, uint32_t members)
{
    const unsigned long long before = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return before == members - 1;
}

struct SumArgs {
    unsigned long long* counters;   // [1 + kMaxGroups] * kCounterStride: the top counter, then one per group
    double* partial;                // [kSums][workers]
    double* group_partial;          // [kSums][groups]
    float* stats;
    float* cost;
    uint32_t workers, groups;
    int accumulate;
};

// Everything the workers exchange goes through device-scope atomic accesses, which are performed at
// the memory side of the caches.  This waits until those the calling wave has issued so far have
// been acknowledged from there, and keeps the compiler from moving memory accesses across it.  (A
// release fence of device scope would also do, but it writes back the whole L2 of the XCD, which costs
// a launch of this size a hundred microseconds; a fence of workgroup scope waits for nothing, since
// the waves of a workgroup share their first-level cache.)
__device__ __forceinline__ void performed()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ double coherent_load(const double* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sums of `members` (at most 256) consecutive values of three statistics, for the wave that calls it:
// wave w of the workgroup takes statistics 3w, 3w + 1, 3w + 2 of src[statistic][stride].  Up to four
// values per lane, all fetched at once (one trip to memory), added lane by lane and then by the
// wave's butterfly: the same additions in the same order whatever the values, so the sums do not
// depend on which workgroup forms them.
__device__ __forceinline__ void add_up(const double* src, uint32_t stride, uint32_t first, uint32_t members,
                                       double (&sums)[3])
{
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    constexpr int kPerLane = kGroup / kWave;
    double v[3][kPerLane];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
#pragma unroll
        for (int q = 0; q < kPerLane; ++q) {
            const uint32_t j = lane + q * kWave;
            v[i][q] = j < members ? coherent_load(src + static_cast<size_t>(wave * 3 + i) * stride + first + j) : 0.0;
        }
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        double t = v[i][0];
#pragma unroll
        for (int q = 1; q < kPerLane; ++q) t += v[i][q];
        sums[i] = wave_sum(t);
    }
}

// Called by every thread of head worker `worker` with its sum of statistic threadIdx.x (threads
// 0..kSums-1).  `flag` is one int of LDS, `totals` LDS for kSums doubles.
__device__ __forceinline__ void leave_sums(double total, uint32_t worker, const SumArgs& s, int* flag, double* totals)
{
    static_assert(kSums == 3 * kWaves, "three statistics per wave");
    if (threadIdx.x < kSums)
        __hip_atomic_store(s.partial + static_cast<size_t>(threadIdx.x) * s.workers + worker, total, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    const uint32_t group = worker / kGroup;
    const uint32_t first = group * kGroup;
    const uint32_t members = min(static_cast<uint32_t>(kGroup), s.workers - first);
    unsigned long long* group_counter = s.counters + (1 + group) * kCounterStride;
    if (threadIdx.x == 0) {
        performed();           // the workgroup's sums (stored by lanes of this wave) are out before it is counted
        *flag = arrive(group_counter, members) ? 1 : 0;
    }
    __syncthreads();
    if (!*flag) return;
    // last of its group: the group's sums
    double sums[3];
    add_up(s.partial, s.workers, first, members, sums);
    if (s.groups > 1) {
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < 3; ++i)
                __hip_atomic_store(s.group_partial + static_cast<size_t>(wave * 3 + i) * s.groups + group, sums[i],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            performed();
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            __hip_atomic_store(group_counter, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = arrive(s.counters, s.groups) ? 1 : 0;
        }
        __syncthreads();
        if (!*flag) return;
        // last of all: the totals
        add_up(s.group_partial, s.groups, 0, s.groups, sums);
    }
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int k = wave * 3 + i;
            totals[k] = sums[i];
            if (s.stats) {
                const float v = static_cast<float>(sums[i]);
                s.stats[k] = (s.accumulate ? s.stats[k] : 0.0f) + v;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s.cost) {
            // the cost is the sum of the four squared-delta statistics, added in double
            const float v = static_cast<float>(((totals[8] + totals[9]) + totals[10]) + totals[11]);
            *s.cost = (s.accumulate ? *s.cost : 0.0f) + v;
        }
        // the counter this workgroup was the last to arrive at is free for the next launch
        __hip_atomic_store(s.groups > 1 ? s.counters : group_counter, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- training pass: persistent head workgroups + class decode stream in one grid ---------------
// The head tiles are instruction bound and the class stream is bandwidth bound, so they run side
// by side: the first `head_workers` workgroups of the grid (dispatched first, a few per compute
// unit) walk the head tiles with a stride, every other workgroup decodes one vector per lane of the
// class rows.  Every delta element belongs to exactly one head tile and every class probability to
// exactly one stream lane, so nothing in the grid waits for anything else in it.
struct TrainArgs {
    HeadArgs head;
    SumArgs sums;
    ClassRuns runs;
    uint32_t head_workers;
};

// FUSED: raw logits in, the class stream decodes them.  !FUSED (the reference's yoloLossGpu
// argument list): the head is already decoded and the grid consists of head workers only.
template<bool FUSED, int L, int V, bool NT>
__global__ __launch_bounds__(kBlock, 4) void yolo_train_kernel(TrainArgs a, YoloParams p, YoloTables tb)
{
    __shared__ TruthSlot tile[kTruthTile];
    __shared__ float pair_iou[kBlock];
    __shared__ double wave_sums[kSums][kWaves];
    __shared__ int flag;
    static_assert(kMaxGroups <= kGroup && kGroup % kWave == 0, "a wave adds up a group");
    if (!FUSED || blockIdx.x < a.head_workers) {
        // the head workers are the long pole of the launch: they go first wherever a SIMD has the choice
        __builtin_amdgcn_s_setprio(3);
        // one sum per worker and statistic, over its tiles in walking order
        double total = 0.0;
        for (uint32_t t = blockIdx.x; t < p.blocks; t += a.head_workers) {
            total += head_tile<FUSED, L, NT>(t, a.head, p, tb, tile, pair_iou, wave_sums);
            __syncthreads();      // wave_sums is read by the first lanes until here
        }
        // the truth tile is free now: it carries the totals from the waves to the cost
        leave_sums(total, blockIdx.x, a.sums, &flag, reinterpret_cast<double*>(tile));
        return;
    }
    if constexpr (FUSED) {
        if constexpr (V == 4) {
            class_stream_block<NT>(a.head.in, a.head.out, a.runs, blockIdx.x - a.head_workers);
        } else {
            // pointers that are not 16-byte aligned: one element per lane
            const uint32_t e = (blockIdx.x - a.head_workers) * kBlock + threadIdx.x;
            if (e >= a.runs.elems) return;
            uint32_t run, at;
            a.runs.by_run_len.divmod(e, run, at);
            const size_t where = static_cast<size_t>(run) * a.runs.run_stride + a.runs.first + at;
            a.head.out[where] = sigmoid_fast(a.head.in[where]);
        }
    }
}

}  // namespace one_launch

// ==========================================================================================
// The training pass in TWO launches, for large heads, whose time is the class stream's: eight
// waves per SIMD for the stream (the head tile squeezed into 64 registers beside it), the class
// stream also writes the zero class deltas, the head tiles leave one int per slot saying what
// supervises it, and a second, small kernel writes the class deltas of those few slots and adds
// up the sums.
// ==========================================================================================
namespace two_launch {

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
        // Both boxes are centred on the origin, where DarkBox's rectangle intersection reduces to
        // min(w) * min(h) exactly: ordered by left edge the wider box comes first, its overlap bound
        // W - (W/2 - n/2) is never below the narrower width n, and the negative-left test
        // (-W/2 + W < -n/2) is false.  The IoU is then formed as box_iou forms it.
        float ba = -FLT_MAX;
        int bi = 0;
        const bool truth_empty = empty;
        const float ab = box.w * box.h;
        for (int a = 0; a < p.anchor_count; ++a) {
            const float cw = p.anchors_rel[2 * a], ch = p.anchors_rel[2 * a + 1];
            const bool none = truth_empty | (cw <= 0.0f) | (ch <= 0.0f);
            const float inter = none ? 0.0f : fminf(cw, box.w) * fminf(ch, box.h);
            const float aa = cw * ch;
            float uni = aa + ab;
            uni = uni - inter;
            const bool some = (uni > 0.0f) & (inter > 0.0f);
            const float q = inter / (some ? uni : 1.0f);
            const float iou = some ? q : 0.0f;
            const bool better = iou > ba;
            ba = better ? iou : ba;
            bi = better ? a : bi;
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

constexpr int kTruthUnroll = 4;

// Returns, in threads 0..kSums-1, the tile's sum of statistic threadIdx.x.
template<bool FUSED>
__device__ __forceinline__ double head_tile(const uint32_t head_block, const HeadArgs& a, const YoloParams& p,
                                          const YoloTables& tb, TruthSlot* tile, double (*wave_sums)[kWaves])
{
    const float* __restrict__ in = a.in;
    float* __restrict__ out = a.out;
    float* __restrict__ delta = a.delta;
    uint32_t bn, tile_id, b, n;
    p.by_tiles.divmod(head_block, bn, tile_id);
    p.by_masks.divmod(bn, b, n);
    const int cell = tile_id * kBlock + threadIdx.x;
    const bool live = cell < p.area;
    const int area = p.area;
    const int entries = p.classes + 5;
    const size_t base = (static_cast<size_t>(bn) * entries) * area + (live ? cell : 0);

    // issued first, used last: the truth count and this lane's truth do not depend on each other
    // a count beyond the table's rows must not read past them
    const int count = min(a.truth_counts[b], p.max_truth);
    const float* image_truths = a.truths + static_cast<size_t>(b) * p.max_truth * 5;

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
    // the host-built table says whether something supervises this slot: asked for with the head rows
    // (it is needed after the sweep, where it would be a trip to memory of its own)
    int table_cls = -1;
    if constexpr (!FUSED) {
        if (live) table_cls = tb.assigned_classes[static_cast<size_t>(bn) * area + cell];
    }
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
    // an empty prediction overlaps nothing: park it where every overlap test fails
    const float pl = pred_empty ? INFINITY : pred.x - pred.w / 2.0f, pt = pred.y - pred.h / 2.0f;

    // Sweep the image's truths through LDS: best IoU (strict >, first wins) and, in the fused
    // form, the truths that claim this slot as their positive (the last one writes the delta).
    // IoU is never negative, so "first wins from the lowest float" is: start at truth 0 with 0.
    float best = 0.0f;
    int best_k = count > 0 ? 0 : -1;
    int pos_cls = -1, pos_anchor = mask_anchor;
    Box pos_box{ 0, 0, 0, 0 };
    float st_iou = 0, st_r50 = 0, st_r75 = 0, st_cat = 0, st_obj = 0, st_count = 0;
    const int my_slot = live ? static_cast<int>(n) * area + cell : -2;

    for (int t0 = 0; t0 < count; t0 += kTruthTile) {
        const int t = t0 + threadIdx.x;
        __syncthreads();       // the previous tile (or the previous head tile of this workgroup) is done with
        if (t < count) tile[threadIdx.x] = make_truth_slot<FUSED>(image_truths + 5 * static_cast<size_t>(t), p);
        __syncthreads();
        const int tn = min(kTruthTile, count - t0);
        // kTruthUnroll truths per step: their overlap tests are independent and interleave; the
        // ordered part (best so far, claims) follows in truth order.  Steps past the last truth
        // re-read it with an empty overlap and no target.
        for (int k0 = 0; k0 < tn; k0 += kTruthUnroll) {
            float inter[kTruthUnroll], tw[kTruthUnroll], th[kTruthUnroll], iou[kTruthUnroll];
            int target[kTruthUnroll];
            bool touch = false, claimed = false;
#pragma unroll
            for (int u = 0; u < kTruthUnroll; ++u) {
                const bool real = k0 + u < tn;
                const int k = real ? k0 + u : tn - 1;
                const float4 r = *reinterpret_cast<const float4*>(&tile[k].left);
                target[u] = real ? tile[k].target : -1;
                tw[u] = r.z; th[u] = r.w;
                const float ov = rect_overlap(pl, pt, pred.w, pred.h, r.x, r.y, r.z, r.w);
                inter[u] = real ? ov : 0.0f;
                touch = touch | (inter[u] > 0.0f);
                claimed = claimed | (target[u] == my_slot);
            }
            // most steps touch nothing in the whole wave: no divisions then
            if (__ballot(touch)) {
#pragma unroll
                for (int u = 0; u < kTruthUnroll; ++u) iou[u] = overlap_ratio(inter[u], pred.w, pred.h, tw[u], th[u]);
#pragma unroll
                for (int u = 0; u < kTruthUnroll; ++u) {
                    const bool better = iou[u] > best;
                    best = better ? iou[u] : best;
                    best_k = better ? t0 + k0 + u : best_k;
                }
            } else {
#pragma unroll
                for (int u = 0; u < kTruthUnroll; ++u) iou[u] = 0.0f;
            }
            if constexpr (FUSED) {
                if (__ballot(claimed)) {
#pragma unroll
                    for (int u = 0; u < kTruthUnroll; ++u) {
                        if (target[u] == my_slot) {
                            // every claiming truth is counted (include/YoloLayer.h:480-507); the claimed
                            // slot's anchor is this mask's, so iou[u] is the IoU the CPU layer records
                            const TruthSlot& ts = tile[k0 + u];
                            pos_cls = ts.cls;
                            pos_box = Box{ ts.x, ts.y, ts.w, ts.h };
                            st_cat += fminf(1.0f, class_prob<FUSED>(in, base, ts.cls, area, p.classes));
                            st_iou += iou[u];
                            if (iou[u] > .5f) st_r50 += 1.0f;
                            if (iou[u] > .75f) st_r75 += 1.0f;
                            st_obj += so;
                            st_count += 1.0f;
                        }
                    }
                }
            }
        }
    }

    if constexpr (!FUSED) {
        if (live) {
            const size_t slot = static_cast<size_t>(bn) * area + cell;
            const int acls = table_cls;
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
                st_cat = fminf(1.0f, class_prob<FUSED>(in, base, acls, area, p.classes));
            }
        }
    }

    // region decision (include/YoloLayer.h:531-545), then the positive override (480-497)
    float d_obj = 0.0f;
    int cls = -1;            // class the dense class delta is written for, -1: zeros
    BoxDelta bd{ { 0, 0, 0, 0 } };
    float c_box = 0, c_obj = 0, c_noobj = 0;
    if (live) {
        const bool have_best = best_k >= 0;
        if (!have_best || best < p.ignore_thresh) d_obj = p.noobject_scale * (0.0f - so);
        if (have_best && best > p.truth_thresh) {
            const float* g = image_truths + 5 * static_cast<size_t>(best_k);
            d_obj = p.object_scale * (1.0f - so);
            cls = static_cast<int>(g[4]);
            bd = box_delta(Box{ g[0], g[1], g[2], g[3] }, sx, sy, rw, rh, i, j, aw, ah, p);
            // deltaYoloClass also feeds the class-probability statistic on this path
            if constexpr (FUSED) st_cat += fminf(1.0f, class_prob<FUSED>(in, base, cls, area, p.classes));
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
        a.decision[static_cast<size_t>(bn) * area + cell] = cls;
    }

    // Workgroup sums.  The objectness sum and the no-object cost exist for every slot: pairwise
    // over the wave.  Everything else is non-zero only at supervised slots, which most waves never
    // see: their lanes are visited one by one, in lane order.  The class deltas are zero except at
    // those slots too; the wave takes their cost together, one class row per lane, from the
    // probabilities the class stream writes (the same function of the same logits).
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const float dense_obj = wave_sum_pairwise(live ? so : 0.0f);
    const float dense_noobj = wave_sum_pairwise(c_noobj);
    const float sparse[9] = { st_iou, st_r50, st_r75, st_cat, st_obj, st_count, st_count, c_box, c_obj };
    constexpr int slot_of[9] = { 0, 1, 2, 3, 4, 6, 7, 8, 9 };
    double acc[9] = { 0, 0, 0, 0, 0, 0, 0, 0, 0 };
    double class_cost = 0.0;
    unsigned long long todo = __ballot(cls >= 0 || st_count != 0.0f);
    while (todo) {
        const int src_lane = __builtin_ctzll(todo);
        todo &= todo - 1;
#pragma unroll
        for (int k = 0; k < 9; ++k)
            acc[k] += static_cast<double>(__shfl(sparse[k], src_lane, kWave));
        const int s_cls = __shfl(cls, src_lane, kWave);
        if (s_cls >= 0) {
            const int s_cell = __shfl(cell, src_lane, kWave);
            const float* rows = in + (static_cast<size_t>(bn) * entries + 5) * area + s_cell;
            float sq = 0.0f;
            for (int c = lane; c < p.classes; c += kWave) {
                const float v = rows[static_cast<size_t>(c) * area];
                const float prob = FUSED ? sigmoid_fast(v) : v;
                const float t = (c == s_cls) ? 1.0f : 0.0f;
                const float d = p.class_scale * (t - prob);
                sq += d * d;
            }
            class_cost += static_cast<double>(wave_sum_pairwise(sq));
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int k = 0; k < 9; ++k) wave_sums[slot_of[k]][wave] = acc[k];
        wave_sums[5][wave] = static_cast<double>(dense_obj);
        wave_sums[10][wave] = static_cast<double>(dense_noobj);
        wave_sums[11][wave] = class_cost;
    }
    __syncthreads();
    double total = 0.0;
    if (threadIdx.x < kSums) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total += wave_sums[threadIdx.x][w];
    }
    return total;
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

// ---- class sweep: decode + dense class delta; the first workgroups add up the head sums --------
struct ClassArgs {
    const float* in;       // the decoded head
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

// statistic k (k < 12) or the cost (k == 12, slots 8..11) over all head workgroups, fixed order
__device__ __forceinline__ void finish_statistic(int k, const ClassArgs& a, double* slots)
{
    const int first = k < 12 ? k : 8, last = k < 12 ? k : 11;
    double s = 0.0;
    for (int kk = first; kk <= last; ++kk) {
        const double* src = a.partial + static_cast<size_t>(kk) * a.head_blocks;
        // four loads in flight per lane; the order of the additions does not depend on it
        for (uint32_t j = threadIdx.x; j < a.head_blocks; j += 4 * kBlock) {
            double v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = j + u * kBlock < a.head_blocks ? src[j + u * kBlock] : 0.0;
#pragma unroll
            for (int u = 0; u < 4; ++u) s += v[u];
        }
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

// ---- fused pass: persistent head workgroups + class decode stream in one grid ------------------
// The head tiles are instruction bound and the class stream is bandwidth bound, so they run side
// by side: the first `head_workers` workgroups of the grid (dispatched first, a few per compute
// unit) walk the head tiles with a stride, every other workgroup decodes one vector per
// lane of the class rows and writes a zero class delta.  The few supervised slots get their class
// delta from yolo_patch_kernel afterwards, so nothing in this grid waits for anything else in it.
struct FusedArgs {
    HeadArgs head;
    ClassSpace space;
    uint32_t head_workers;
};

// FUSED: raw logits in, the class stream decodes them.  !FUSED (the reference's yoloLossGpu
// argument list): the head is already decoded and the class stream only writes the zero delta.
// Eight waves per SIMD (at most 64 vector registers): the class stream needs the occupancy.
template<bool FUSED, int V, bool NT>
__global__ __launch_bounds__(kBlock, 8) void yolo_fused_kernel(FusedArgs a, YoloParams p, YoloTables tb)
{
    __shared__ TruthSlot tile[kTruthTile];
    __shared__ double wave_sums[kSums][kWaves];
    if (blockIdx.x < a.head_workers) {
        // one sum per worker and statistic, over its tiles in walking order
        double total = 0.0;
        for (uint32_t t = blockIdx.x; t < p.blocks; t += a.head_workers) {
            total += head_tile<FUSED>(t, a.head, p, tb, tile, wave_sums);
            __syncthreads();      // wave_sums is read by the first lanes until here
        }
        if (threadIdx.x < kSums)
            a.head.partial[static_cast<size_t>(threadIdx.x) * a.head_workers + blockIdx.x] = total;
        return;
    }
    const uint32_t e = ((blockIdx.x - a.head_workers) * kBlock + threadIdx.x) * V;
    if (e >= a.space.elems) return;
    uint32_t bn, c, cell;
    a.space.locate(e, bn, c, cell);
    const size_t at = a.space.offset(bn, c, cell);
    Pack<V> zero;
#pragma unroll
    for (int k = 0; k < V; ++k) zero.v[k] = 0.0f;
    if constexpr (FUSED) {
        const Pack<V> x = ld<V, NT>(a.head.in, at);
        Pack<V> prob;
#pragma unroll
        for (int k = 0; k < V; ++k) prob.v[k] = sigmoid_fast(x.v[k]);
        st<V, NT>(a.head.out, at, prob);
    }
    st<V, NT>(a.head.delta, at, zero);
}

// One lane per slot finds the supervised ones; a wave then writes the class delta of each of its
// supervised slots together (one class row per lane) from the probabilities the fused pass wrote.
// The first workgroups also add up the head sums.
struct PatchArgs {
    ClassArgs cls;        // in = the decoded head; out unused
    uint32_t slots;       // batch * masks * area
    int classes;
};

__global__ __launch_bounds__(kBlock) void yolo_patch_kernel(PatchArgs a)
{
    __shared__ double slots[kBlock / kWave];
    const uint32_t slot = blockIdx.x * kBlock + threadIdx.x;
    const int cls = slot < a.slots ? a.cls.decision[slot] : -1;
    const int lane = threadIdx.x & (kWave - 1);
    unsigned long long todo = __ballot(cls >= 0);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const uint32_t s_slot = __shfl(slot, src, kWave);
        const int s_cls = __shfl(cls, src, kWave);
        uint32_t bn, cell;
        a.cls.space.by_area.divmod(s_slot, bn, cell);
        for (int c = lane; c < a.classes; c += kWave) {
            const size_t at = a.cls.space.offset(bn, c, cell);
            const float t = (c == s_cls) ? 1.0f : 0.0f;
            a.cls.delta[at] = a.cls.class_scale * (t - a.cls.in[at]);
        }
    }
    if (blockIdx.x < 13) finish_statistic(blockIdx.x, a.cls, slots);
}

}  // namespace two_launch

// ==========================================================================================
// All heads of a model in one pass.  A model runs each of its heads where it sits in the graph
// (include/Model.h:1740-1759, include/YoloLayer.h:164-239 of the reference), but nothing reads a
// head's delta or cost before the backward pass, so the heads can all wait for the last one: one grid
// whose head workers walk the tiles of every head and whose class stream covers every head's class
// rows, then one small kernel for the supervised slots' class deltas and the sums of every head.  A
// small head alone is bound by the chain of steps of one head tile, with most of the machine idle;
// here that chain runs under the class stream of the large head.  The two-launch form's kernels, per
// head: the results per head are those of pxh_yolo_forward_train on that head.
// ==========================================================================================
namespace all_heads {

constexpr int kMaxHeads = 4;

struct HeadPart {
    two_launch::HeadArgs head;
    two_launch::ClassSpace space;
    uint32_t head_workers;      // persistent workgroups that walk this head's tiles
    uint32_t first_worker;      // ... and the first of them in the grid
    uint32_t class_blocks;      // workgroups of the class stream on this head
    uint32_t first_class_block; // ... counted from the end of the head workers
    int vec;                    // 128-bit accesses on this head's class rows
    int nt;
};

struct HeadsArgs {
    int count;
    uint32_t workers;           // head workers of all heads
    HeadPart part[kMaxHeads];
    YoloParams p[kMaxHeads];
};

// The head that workgroup `index` of a run of workgroups belongs to: the last one whose first
// workgroup is not beyond it (`firsts` ascend).
template<typename First>
__device__ __forceinline__ int head_of(int count, uint32_t index, First&& first)
{
    int h = 0;
#pragma unroll
    for (int k = 1; k < kMaxHeads; ++k)
        if (k < count && index >= first(k)) h = k;
    return h;
}

// Block `block` of a head's class stream, one vector per lane: logit -> probability -> `out`, and the
// zero class delta.  (One read and two written streams: a plain kernel of that mix moves 5.9 TB/s on
// this part against 6.6 for a copy; two or four vectors per lane were slower, here and there.)
template<int V, bool NT>
__device__ __forceinline__ void class_block(const HeadPart& part, uint32_t block)
{
    const uint32_t e = (block * kBlock + threadIdx.x) * V;
    if (e >= part.space.elems) return;
    uint32_t bn, c, cell;
    part.space.locate(e, bn, c, cell);
    const size_t at = part.space.offset(bn, c, cell);
    Pack<V> zero;
#pragma unroll
    for (int k = 0; k < V; ++k) zero.v[k] = 0.0f;
    const Pack<V> x = ld<V, NT>(part.head.in, at);
    Pack<V> prob;
#pragma unroll
    for (int k = 0; k < V; ++k) prob.v[k] = sigmoid_fast(x.v[k]);
    st<V, NT>(part.head.out, at, prob);
    st<V, NT>(part.head.delta, at, zero);
}

__global__ __launch_bounds__(kBlock, 8) void yolo_heads_kernel(HeadsArgs a)
{
    __shared__ TruthSlot tile[kTruthTile];
    __shared__ double wave_sums[kSums][kWaves];
    if (blockIdx.x < a.workers) {
        const int h = head_of(a.count, blockIdx.x, [&](int k) { return a.part[k].first_worker; });
        const HeadPart& part = a.part[h];
        const YoloParams& p = a.p[h];
        const uint32_t worker = blockIdx.x - part.first_worker;
        // one sum per worker and statistic, over its tiles in walking order
        double total = 0.0;
        for (uint32_t t = worker; t < p.blocks; t += part.head_workers) {
            total += two_launch::head_tile<true>(t, part.head, p, YoloTables{}, tile, wave_sums);
            __syncthreads();      // wave_sums is read by the first lanes until here
        }
        if (threadIdx.x < kSums) part.head.partial[static_cast<size_t>(threadIdx.x) * part.head_workers + worker] = total;
        return;
    }
    const uint32_t block = blockIdx.x - a.workers;
    const int h = head_of(a.count, block, [&](int k) { return a.part[k].first_class_block; });
    const HeadPart& part = a.part[h];
    const uint32_t local = block - part.first_class_block;
    if (part.vec) {
        if (part.nt) class_block<4, true>(part, local);
        else class_block<4, false>(part, local);
    } else {
        class_block<1, false>(part, local);
    }
}

struct PatchPart {
    two_launch::ClassArgs cls;      // in = the decoded head
    uint32_t slots;                 // batch * masks * area
    uint32_t first_block;           // of this head's slots in the grid
    int classes;
};

struct PatchHeadsArgs {
    int count;
    PatchPart part[kMaxHeads];
};

// The supervised slots' class deltas of every head (one lane per slot finds them, a wave writes each
// slot's class rows together); the first 13 workgroups per head also add up that head's sums.
__global__ __launch_bounds__(kBlock) void yolo_heads_patch_kernel(PatchHeadsArgs a)
{
    __shared__ double slots[kBlock / kWave];
    {
        const int h = head_of(a.count, blockIdx.x, [&](int k) { return a.part[k].first_block; });
        const PatchPart& part = a.part[h];
        const uint32_t slot = (blockIdx.x - part.first_block) * kBlock + threadIdx.x;
        const int cls = slot < part.slots ? part.cls.decision[slot] : -1;
        const int lane = threadIdx.x & (kWave - 1);
        unsigned long long todo = __ballot(cls >= 0);
        while (todo) {
            const int src = __builtin_ctzll(todo);
            todo &= todo - 1;
            const uint32_t s_slot = __shfl(slot, src, kWave);
            const int s_cls = __shfl(cls, src, kWave);
            uint32_t bn, cell;
            part.cls.space.by_area.divmod(s_slot, bn, cell);
            for (int c = lane; c < part.classes; c += kWave) {
                const size_t at = part.cls.space.offset(bn, c, cell);
                const float t = (c == s_cls) ? 1.0f : 0.0f;
                part.cls.delta[at] = part.cls.class_scale * (t - part.cls.in[at]);
            }
        }
    }
    if (blockIdx.x < 13u * a.count) two_launch::finish_statistic(blockIdx.x % 13, a.part[blockIdx.x / 13].cls, slots);
}

}  // namespace all_heads

// ---------------------------------------------------------------- detections
// Thresholded compaction of a decoded head (include/YoloLayer.h:601-698): one lane per slot; a slot
// whose objectness passes walks its class rows, and all lanes of a workgroup that found detections
// in the same class step reserve their output places with one atomic between them: the counter is
// one address for the whole grid, takes about 15 ns per atomic, and at one atomic per wave that
// was most of the kernel's time when half the slots pass.  The records carry their position in the
// reference's emission order, so sorting by it restores that order.
struct DetectArgs {
    const float* pred;
    pxh_detection* out;
    int* count;
    int capacity;
    float threshold;
    int image_width, image_height;    // > 0: letterbox-corrected pixel boxes
    uint32_t slots;                   // batch * masks * area
    uint32_t order_base;              // added to every record's emission order
    FastDiv by_area;
};

constexpr int kDetectBlock = 512;

__global__ __launch_bounds__(kDetectBlock) void yolo_detect_kernel(DetectArgs a, YoloParams p)
{
    __shared__ int wave_first[kDetectBlock / kWave];
    __shared__ int group_first;
    const uint32_t t = blockIdx.x * kDetectBlock + threadIdx.x;
    const bool live = t < a.slots;
    const uint32_t slot = live ? t : 0;
    uint32_t bn, cell, b, n;
    a.by_area.divmod(slot, bn, cell);
    p.by_masks.divmod(bn, b, n);
    const int area = p.area;
    const size_t base = static_cast<size_t>(bn) * (p.classes + 5) * area + cell;
    const float objectness = live ? a.pred[base + 4 * static_cast<size_t>(area)] : -INFINITY;
    bool pass = live && !(objectness < a.threshold);
    float bx = 0, by = 0, bw = 0, bh = 0;
    if (pass) {
        uint32_t row, col;
        p.by_width.divmod(cell, row, col);
        const int anchor = p.masks[n];
        const float p0 = a.pred[base], p1 = a.pred[base + area], p2 = a.pred[base + 2 * static_cast<size_t>(area)],
                    p3 = a.pred[base + 3 * static_cast<size_t>(area)];
        if (a.image_width > 0 && a.image_height > 0) {
            const int w = a.image_width, h = a.image_height;
            const int netW = p.net_width, netH = p.net_height;
            int newW, newH;
            if ((static_cast<float>(netW) / w) < (static_cast<float>(netH) / h)) {
                newW = netW;
                newH = (h * netW) / w;
            } else {
                newH = netH;
                newW = (w * netH) / h;
            }
            float x = (static_cast<float>(col) + p0) / static_cast<float>(p.width);
            x = (x - static_cast<float>(netW - newW) / 2.0f / static_cast<float>(netW)) /
                (static_cast<float>(newW) / static_cast<float>(netW));
            float y = (static_cast<float>(row) + p1) / static_cast<float>(p.height);
            y = (y - static_cast<float>(netH - newH) / 2.0f / static_cast<float>(netH)) /
                (static_cast<float>(newH) / static_cast<float>(netH));
            float width = expf(p2) * p.anchors[2 * anchor] / static_cast<float>(netW);
            width *= static_cast<float>(netW) / static_cast<float>(newW);
            float height = expf(p3) * p.anchors[2 * anchor + 1] / static_cast<float>(netH);
            height *= static_cast<float>(netH) / static_cast<float>(newH);
            const int left = max(0, static_cast<int>((x - width / 2) * static_cast<float>(w)));
            const int right = min(w - 1, static_cast<int>((x + width / 2) * static_cast<float>(w)));
            const int top = max(0, static_cast<int>((y - height / 2) * static_cast<float>(h)));
            const int bottom = min(h - 1, static_cast<int>((y + height / 2) * static_cast<float>(h)));
            bx = static_cast<float>(left); by = static_cast<float>(top);
            bw = static_cast<float>(right - left); bh = static_cast<float>(bottom - top);
        } else {
            const float x = (static_cast<float>(col) + p0) / static_cast<float>(p.width);
            const float y = (static_cast<float>(row) + p1) / static_cast<float>(p.height);
            bw = expf(p2) * p.anchors[2 * anchor] / static_cast<float>(p.net_width);
            bh = expf(p3) * p.anchors[2 * anchor + 1] / static_cast<float>(p.net_height);
            // DarkBox::rect(): the corner falls back to the centre for a non-positive size
            bx = bw > 0.0f ? x - bw / 2.0f : x;
            by = bh > 0.0f ? y - bh / 2.0f : y;
        }
    }
    if (!__syncthreads_or(pass)) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint32_t order0 = ((b * static_cast<uint32_t>(area) + cell) * p.mask_count + n) * p.classes;
    const float* rows = a.pred + base + 5 * static_cast<size_t>(area);
    // 128 classes at a time: each lane notes its hits in a bit mask, the workgroup reserves the
    // places of all of them with ONE atomic, then every lane writes its records one after the other.
    // The class rows are read 32 at a time with their loads in flight together (one after the other
    // they cost a memory latency each, the larger part of the kernel's time when many slots pass),
    // and read again, from the cache, for the words that hold a hit.  Keeping 64 of them in registers
    // over the reservation instead was slower: 171 registers, two waves per SIMD.
    constexpr int kWords = 4;
    for (int j0 = 0; j0 < p.classes; j0 += 32 * kWords) {
        uint32_t hits[kWords];
        int mine = 0;
#pragma unroll
        for (int w = 0; w < kWords; ++w) {
            hits[w] = 0u;
            const int first = j0 + 32 * w;
            const int rows_here = min(32, p.classes - first);
            if (pass && rows_here > 0) {
                float v[32];
#pragma unroll
                for (int k = 0; k < 32; ++k) v[k] = rows[static_cast<size_t>(first + min(k, rows_here - 1)) * area];
#pragma unroll
                for (int k = 0; k < 32; ++k) {
                    if (k < rows_here && objectness * v[k] >= a.threshold) {
                        hits[w] |= 1u << k;
                        ++mine;
                    }
                }
            }
        }
        int upto = mine;      // inclusive prefix sum over the lanes
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int up = __shfl_up(upto, off, kWave);
            if (lane >= off) upto += up;
        }
        if (j0 > 0) __syncthreads();      // the previous step's places have been read
        if (lane == kWave - 1) wave_first[wave] = upto;
        __syncthreads();
        if (threadIdx.x == 0) {
            int sum = 0;
#pragma unroll
            for (int w = 0; w < kDetectBlock / kWave; ++w) {
                const int n_w = wave_first[w];
                wave_first[w] = sum;
                sum += n_w;
            }
            group_first = sum ? atomicAdd(a.count, sum) : 0;
        }
        __syncthreads();
        int at = group_first + wave_first[wave] + upto - mine;
#pragma unroll
        for (int w = 0; w < kWords; ++w) {
            if (!hits[w]) continue;
            if (at >= a.capacity) {
                at += __builtin_popcount(hits[w]);
                continue;
            }
            const int first = j0 + 32 * w;
            const int rows_here = min(32, p.classes - first);
            float v[32];
#pragma unroll
            for (int k = 0; k < 32; ++k) v[k] = rows[static_cast<size_t>(first + min(k, rows_here - 1)) * area];
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                if (!((hits[w] >> k) & 1u)) continue;
                if (at < a.capacity) {
                    pxh_detection d;
                    d.x = bx; d.y = by; d.w = bw; d.h = bh;
                    d.prob = objectness * v[k];
                    d.batch = static_cast<int>(b);
                    d.class_index = first + k;
                    d.order = a.order_base + order0 + first + k;
                    a.out[at] = d;
                }
                ++at;
            }
        }
    }
}

// Head tiles of kBlock / lanes cells each.
void set_lanes_per_slot(YoloParams& p, int lanes)
{
    const int cells = kBlock / lanes;
    const int tiles = (p.area + cells - 1) / cells;
    p.by_tiles = FastDiv(tiles);
    p.blocks = static_cast<uint32_t>(p.batch) * p.mask_count * tiles;
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
    p.by_masks = FastDiv(mask_count);
    p.by_width = FastDiv(width);
    p.by_anchors = FastDiv(anchor_count);
    p.by_area = FastDiv(static_cast<uint32_t>(p.area));
    set_lanes_per_slot(p, 1);
    return PXH_OK;
}

size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }

namespace one_launch {

// workspace: [12][workers] doubles | [12][groups] doubles
struct YoloWorkspace {
    double* partial;
    double* group_partial;
};

size_t yolo_workspace_bytes()
{
    return align256(static_cast<size_t>(kMaxWorkers) * kSums * sizeof(double)) +
           align256(static_cast<size_t>(kMaxGroups) * kSums * sizeof(double));
}

YoloWorkspace carve(void* ws)
{
    YoloWorkspace w;
    char* c = static_cast<char*>(ws);
    w.partial = reinterpret_cast<double*>(c);
    c += align256(static_cast<size_t>(kMaxWorkers) * kSums * sizeof(double));
    w.group_partial = reinterpret_cast<double*>(c);
    return w;
}

// The arrival counters of the workspace at `ws` on the current device: a set of g_arrival_counters,
// handed out the first time the address is seen and kept for it.  Launches that may overlap have
// workspaces of their own, hence sets of their own.  When every set is taken, the address that has
// gone unused longest among those last used on `stream` gives up its set: the launch that used it
// is ordered before this one, and its counters are back at zero when it has run.  (A graph captured
// with a workspace bakes its set in: workspaces of captured calls should be long-lived ones.)
// kNoCounterSet: every set belongs to an address last used on another stream.
constexpr int kNoCounterSet = -1000;      // internal, never returned to a caller of the library

int counters_for(const char* who, const void* ws, hipStream_t stream, unsigned long long** out)
{
    constexpr int kDevices = 64;
    struct Owner {
        const void* ws;
        hipStream_t stream;
        unsigned long long last_use;
    };
    struct PerDevice {
        unsigned long long* base = nullptr;
        unsigned long long uses = 0;
        std::vector<Owner> owners;      // owners[i] holds set i
    };
    static std::mutex mutex;
    static PerDevice devices[kDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kDevices) {
        set_error("%s: no usable current device (%s)", who, hipGetErrorString(e));
        return PXH_ERR_WORKSPACE;
    }
    std::lock_guard<std::mutex> lock(mutex);
    PerDevice& d = devices[dev];
    if (!d.base) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_arrival_counters));
        if (e != hipSuccess || !p) {
            set_error("%s: hipGetSymbolAddress(arrival counters): %s", who, hipGetErrorString(e));
            return e != hipSuccess ? static_cast<int>(e) : PXH_ERR_WORKSPACE;
        }
        d.base = static_cast<unsigned long long*>(p);
    }
    size_t set = 0;
    while (set < d.owners.size() && d.owners[set].ws != ws) ++set;
    if (set == d.owners.size()) {
        if (set < static_cast<size_t>(kCounterSets)) {
            d.owners.push_back(Owner{ ws, stream, 0 });
        } else {
            size_t oldest = d.owners.size();
            for (size_t i = 0; i < d.owners.size(); ++i)
                if (d.owners[i].stream == stream && (oldest == d.owners.size() || d.owners[i].last_use < d.owners[oldest].last_use))
                    oldest = i;
            if (oldest == d.owners.size()) return kNoCounterSet;     // the caller takes the form without counters
            set = oldest;
            d.owners[set].ws = ws;
        }
    }
    d.owners[set].stream = stream;
    d.owners[set].last_use = ++d.uses;
    *out = d.base + set * kCountersPerSet * kCounterStride;
    return PXH_OK;
}

// Test hook state: lanes per slot and head workers forced by pxh_debug_yolo_tuning (0 = chosen here).
std::atomic<int> g_forced_lanes{ 0 };
std::atomic<int> g_forced_workers{ 0 };
// Lanes per slot: a head with few slots is bound by the length of one lane's instruction stream and
// gains from spreading a slot's truth sweep over two lanes (measured: 64 x 19^2 and 16 x 38^2, 69 k slots,
// run 12 % faster with two lanes than with one, no faster with four); a head with many slots has
// enough waves to hide it and is cheapest with one lane per slot.
int lanes_per_slot(const YoloParams& p)
{
    const int forced = g_forced_lanes.load();
    if (forced == 1 || forced == 2 || forced == 4) return forced;
    const size_t slots = static_cast<size_t>(p.batch) * p.mask_count * p.area;
    return slots < 200000 ? 2 : 1;
}

// Persistent head workgroups of the fused pass.  A head tile takes about kTileMicros however
// many run side by side, so enough of them are started to be through in the time the class rows
// take to stream, and no more: every one holds wave slots the stream could use.
uint32_t head_workers(uint32_t tiles, double stream_us)
{
    const int forced = g_forced_workers.load();
    uint32_t want;
    if (forced > 0) {
        want = static_cast<uint32_t>(forced);
    } else {
        constexpr double kTileMicros = 22.0;
        double rounds = stream_us * 0.85 / kTileMicros;
        if (rounds < 1.0) rounds = 1.0;
        want = static_cast<uint32_t>(static_cast<double>(tiles) / rounds) + 1;
    }
    if (want > kMaxWorkers) want = kMaxWorkers;
    return want < tiles ? want : tiles;
}

template<bool FUSED, int L>
void launch_training(const TrainArgs& ta, const YoloParams& p, const YoloTables& tb, uint32_t grid, bool vec, bool nt,
                     hipStream_t s)
{
    const dim3 g(grid), b(kBlock);
    if constexpr (!FUSED) {
        if (nt) hipLaunchKernelGGL((yolo_train_kernel<false, L, 1, true>), g, b, 0, s, ta, p, tb);
        else hipLaunchKernelGGL((yolo_train_kernel<false, L, 1, false>), g, b, 0, s, ta, p, tb);
    } else {
        if (vec && nt) hipLaunchKernelGGL((yolo_train_kernel<true, L, 4, true>), g, b, 0, s, ta, p, tb);
        else if (vec) hipLaunchKernelGGL((yolo_train_kernel<true, L, 4, false>), g, b, 0, s, ta, p, tb);
        else hipLaunchKernelGGL((yolo_train_kernel<true, L, 1, false>), g, b, 0, s, ta, p, tb);
    }
}

template<bool FUSED>
int run_training_pass(const char* who, const float* in, float* out, float* delta, const float* truths,
                      const int* truth_counts, YoloParams p, const YoloTables& tb, float* stats, float* cost,
                      int accumulate, void* ws, hipStream_t s)
{
    const YoloWorkspace w = carve(ws);
    ClassRuns runs{};
    runs.run_len = static_cast<uint32_t>(p.classes) * p.area;
    runs.run_stride = static_cast<uint32_t>(p.classes + 5) * p.area;
    runs.first = 5u * p.area;
    const uint32_t slots_per_run = (runs.run_len + 6) / 4;
    runs.by_slots = FastDiv(slots_per_run);
    runs.by_run_len = FastDiv(runs.run_len);
    const uint32_t run_count = static_cast<uint32_t>(p.batch) * p.mask_count;
    runs.total_slots = run_count * slots_per_run;
    runs.elems = run_count * runs.run_len;
    const bool vec = aligned16(in) && aligned16(out);
    const uint32_t class_blocks = !FUSED ? 0
                                  : vec ? (runs.total_slots + kBlock * kClassVectors - 1) / (kBlock * kClassVectors)
                                        : (runs.elems + kBlock - 1) / kBlock;

    const int lanes = lanes_per_slot(p);
    set_lanes_per_slot(p, lanes);
    // class rows: read + decode (the deltas are the head workers' business)
    const double stream_us = static_cast<double>(runs.elems) * 8 / 6.0e6;   // at 6 TB/s
    TrainArgs ta{};
    ta.head = HeadArgs{ in, out, delta, truths, truth_counts, (p.area % 4 == 0 && aligned16(delta)) ? 1 : 0 };
    ta.runs = runs;
    ta.head_workers = FUSED ? head_workers(p.blocks, stream_us) : (p.blocks < kMaxWorkers ? p.blocks : kMaxWorkers);
    int rc = counters_for(who, ws, s, &ta.sums.counters);
    if (rc) return rc;
    ta.sums.partial = w.partial;
    ta.sums.group_partial = w.group_partial;
    ta.sums.stats = stats;
    ta.sums.cost = cost;
    ta.sums.workers = ta.head_workers;
    ta.sums.groups = (ta.head_workers + kGroup - 1) / kGroup;
    ta.sums.accumulate = accumulate;
    const uint32_t grid = ta.head_workers + class_blocks;
    const bool nt = static_cast<size_t>(runs.elems) * (FUSED ? 12 : 4) >= kStreamingBytes;
    switch (lanes) {
    case 1: launch_training<FUSED, 1>(ta, p, tb, grid, vec, nt, s); break;
    case 2: launch_training<FUSED, 2>(ta, p, tb, grid, vec, nt, s); break;
    default: launch_training<FUSED, 4>(ta, p, tb, grid, vec, nt, s); break;
    }
    return check_launch(who);
}

}  // namespace one_launch

namespace two_launch {

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

// Persistent head workgroups of the fused pass.  A head tile takes about kTileMicros however
// many run side by side, so enough of them are started to be through in the time the class rows
// take to stream, and no more: every one holds wave slots the stream could use.
uint32_t head_workers(uint32_t tiles, double stream_us)
{
    constexpr double kTileMicros = 22.0;
    double rounds = stream_us * 0.85 / kTileMicros;
    if (rounds < 1.0) rounds = 1.0;
    uint32_t want = static_cast<uint32_t>(static_cast<double>(tiles) / rounds) + 1;
    return want < tiles ? want : tiles;
}

// The same for the form that starts from a decoded head, whose stream only writes zeros.  A head
// worker holds a workgroup slot for the whole pass, and such a stream is done in a few tens of
// microseconds: beyond about 3.5 workers per compute unit it is starved of slots until the workers
// leave, and the two run one after the other (measured at 64 x 255 x 76^2, 4332 tiles: 900 workers
// 60 us, 1500 workers 77 us, 1900 workers 83 us; at 32 x 255 x 76^2: 39 us against 46 us).  Up to
// 1200 tiles every tile gets its worker: one round of tiles is the shortest the pass can be.
uint32_t head_workers_beside_fill(uint32_t tiles)
{
    return tiles <= 1200u ? tiles : 900u;
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

    ClassArgs ca{};
    ca.in = FUSED ? out : in;      // the decoded head
    ca.delta = delta;
    ca.decision = w.decision;
    ca.partial = w.partial;
    ca.stats = stats;
    ca.cost = cost;
    ca.space = space;
    ca.head_blocks = p.blocks;
    ca.class_scale = p.class_scale;
    ca.accumulate = accumulate;
    const HeadArgs ha{ in, out, delta, truths, truth_counts, w.decision, w.partial };

    const int stream_bytes = FUSED ? 12 : 4;      // per class element: read + decode + zero delta, or the zero delta alone
    const double stream_us = static_cast<double>(space.elems) * stream_bytes / 6.0e6;   // at 6 TB/s
    FusedArgs fa{ ha, space, FUSED ? head_workers(p.blocks, stream_us) : head_workers_beside_fill(p.blocks) };
    if (const int forced = one_launch::g_forced_workers.load(); forced > 0)
        fa.head_workers = static_cast<uint32_t>(forced) < p.blocks ? static_cast<uint32_t>(forced) : p.blocks;
    ca.head_blocks = fa.head_workers;      // one partial sum per worker
    const uint32_t grid = fa.head_workers + class_blocks;
    const bool nt = static_cast<size_t>(space.elems) * stream_bytes >= kStreamingBytes;
    if (vec && nt) hipLaunchKernelGGL((yolo_fused_kernel<FUSED, 4, true>), dim3(grid), dim3(kBlock), 0, s, fa, p, tb);
    else if (vec) hipLaunchKernelGGL((yolo_fused_kernel<FUSED, 4, false>), dim3(grid), dim3(kBlock), 0, s, fa, p, tb);
    else hipLaunchKernelGGL((yolo_fused_kernel<FUSED, 1, false>), dim3(grid), dim3(kBlock), 0, s, fa, p, tb);
    int rc = check_launch(who);
    if (rc) return rc;
    PatchArgs pa{ ca, static_cast<uint32_t>(p.batch) * p.mask_count * p.area, p.classes };
    const uint32_t pgrid = grid_for(pa.slots, kBlock);
    hipLaunchKernelGGL(yolo_patch_kernel, dim3(pgrid < 13 ? 13 : pgrid), dim3(kBlock), 0, s, pa);
    return check_launch(who);
}

}  // namespace two_launch

// Test hook state: the form of the training pass forced by pxh_debug_yolo_tuning (0 = chosen here).
std::atomic<int> g_forced_form{ 0 };

size_t training_workspace_bytes(int batch, int mask_count, int width, int height)
{
    const size_t a = one_launch::yolo_workspace_bytes(), b = two_launch::yolo_workspace_bytes(batch, mask_count, width, height);
    return a > b ? a : b;
}

// One launch where the pass is bound by the head tiles' chain of steps, two where it is bound by the
// class stream (measured on MI355X at 80 classes: below about 110 MB of fused traffic, and below
// about 40 MB for the form that starts from a decoded head, one launch is the faster).
template<bool FUSED>
int run_training_pass(const char* who, const float* in, float* out, float* delta, const float* truths,
                      const int* truth_counts, const YoloParams& p, const YoloTables& tb, float* stats, float* cost,
                      int accumulate, void* ws, hipStream_t s)
{
    const size_t elems = static_cast<size_t>(p.batch) * p.mask_count * (p.classes + 5) * p.area;
    const size_t bytes = FUSED ? elems * 12 : elems * 4 + elems * 20 / static_cast<size_t>(p.classes + 5);
    const int forced = g_forced_form.load();
    const bool one = forced == 1 || (forced != 2 && bytes < (FUSED ? size_t(110) << 20 : size_t(40) << 20));
    if (one) {
        const int rc = one_launch::run_training_pass<FUSED>(who, in, out, delta, truths, truth_counts, p, tb, stats, cost,
                                                            accumulate, ws, s);
        // no arrival counters to be had for this workspace address (see counters_for): nothing was
        // launched, and the form that needs none does the same work
        if (rc != one_launch::kNoCounterSet) return rc;
    }
    YoloParams q = p;
    set_lanes_per_slot(q, 1);
    return two_launch::run_training_pass<FUSED>(who, in, out, delta, truths, truth_counts, q, tb, stats, cost,
                                                accumulate, ws, s);
}

namespace all_heads {

// workspace: per head the two-launch form's [12][head workers] doubles and one int per slot
size_t workspace_bytes(int count, const pxh_yolo_head* heads, int batch)
{
    size_t total = 0;
    for (int h = 0; h < count; ++h)
        total += two_launch::yolo_workspace_bytes(batch, heads[h].mask_count, heads[h].width, heads[h].height);
    return total;
}

int run(const char* who, int count, const pxh_yolo_head* heads, const YoloParams* params, const float* truths,
        const int* truth_counts, void* ws, hipStream_t s)
{
    HeadsArgs a{};
    PatchHeadsArgs pa{};
    a.count = pa.count = count;
    // the class stream of all heads together sets the time the head workers have
    double stream_us = 0.0;
    for (int h = 0; h < count; ++h) {
        const YoloParams& p = params[h];
        stream_us += static_cast<double>(p.batch) * p.mask_count * p.classes * p.area * 12 / 6.0e6;   // at 6 TB/s
    }
    uint64_t tiles_total = 0;
    for (int h = 0; h < count; ++h) tiles_total += params[h].blocks;
    char* at = static_cast<char*>(ws);
    uint32_t workers = 0, class_blocks = 0, patch_blocks = 0;
    for (int h = 0; h < count; ++h) {
        const YoloParams& p = params[h];
        a.p[h] = p;
        const two_launch::YoloWorkspace w = two_launch::carve(at, p);
        at += two_launch::yolo_workspace_bytes(p.batch, p.mask_count, p.width, p.height);
        const two_launch::ClassSpace space{ FastDiv(p.area), FastDiv(p.classes), static_cast<uint32_t>(p.area),
                                            static_cast<uint32_t>(p.classes + 5),
                                            static_cast<uint32_t>(static_cast<size_t>(p.batch) * p.mask_count *
                                                                  p.classes * p.area) };
        HeadPart& part = a.part[h];
        part.head = two_launch::HeadArgs{ heads[h].input, heads[h].output, heads[h].delta, truths, truth_counts,
                                          w.decision, w.partial };
        part.space = space;
        part.head_workers = two_launch::head_workers(p.blocks, stream_us);
        if (const int forced = one_launch::g_forced_workers.load(); forced > 0) {
            // the test hook's figure is for the call: every head gets its share by tiles, one at least
            const uint64_t share = static_cast<uint64_t>(forced) * p.blocks / tiles_total;
            part.head_workers = share < 1 ? 1u : share < p.blocks ? static_cast<uint32_t>(share) : p.blocks;
        }
        part.first_worker = workers;
        workers += part.head_workers;
        part.vec = p.area % 4 == 0 && aligned16(heads[h].input) && aligned16(heads[h].output) && aligned16(heads[h].delta);
        const uint32_t per_block = kBlock * (part.vec ? 4 : 1);
        part.class_blocks = (space.elems + per_block - 1) / per_block;
        part.first_class_block = class_blocks;
        class_blocks += part.class_blocks;
        part.nt = stream_us * 6.0e6 >= static_cast<double>(kStreamingBytes);

        PatchPart& pp = pa.part[h];
        pp.cls.in = heads[h].output;
        pp.cls.delta = heads[h].delta;
        pp.cls.decision = w.decision;
        pp.cls.partial = w.partial;
        pp.cls.stats = heads[h].stats;
        pp.cls.cost = heads[h].cost;
        pp.cls.space = space;
        pp.cls.head_blocks = part.head_workers;
        pp.cls.class_scale = p.class_scale;
        pp.cls.accumulate = 0;
        pp.slots = static_cast<uint32_t>(p.batch) * p.mask_count * p.area;
        pp.classes = p.classes;
        pp.first_block = patch_blocks;
        patch_blocks += grid_for(pp.slots, kBlock);
    }
    a.workers = workers;
    const unsigned long long grid = 1ull * workers + class_blocks;
    if (grid >= (1ull << 31)) {
        set_error("%s: more than 2^31 workgroups in one launch", who);
        return PXH_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(yolo_heads_kernel, dim3(static_cast<unsigned>(grid)), dim3(kBlock), 0, s, a);
    int rc = check_launch(who);
    if (rc) return rc;
    const uint32_t least = 13u * count;
    hipLaunchKernelGGL(yolo_heads_patch_kernel, dim3(patch_blocks < least ? least : patch_blocks), dim3(kBlock), 0, s, pa);
    return check_launch(who);
}

}  // namespace all_heads

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

int pxh_yolo_detections_append(const float* predictions, int batch, const int* host_masks, int mask_count,
                               const int* host_anchors, int anchor_count, int classes, int width, int height,
                               int net_width, int net_height, int image_width, int image_height, float threshold,
                               unsigned order_base, pxh_detection* out, int capacity, int* count, void* stream)
{
    if (!predictions || !host_masks || !host_anchors || !count || (!out && capacity > 0))
        return fail_invalid("pxh_yolo_detections: null pointer");
    if (capacity < 0) return fail_invalid("pxh_yolo_detections: negative capacity");
    YoloParams p{};
    int rc = fill_params("pxh_yolo_detections", p, batch, mask_count, anchor_count, classes, width, height, net_width,
                         net_height, 0, 0.0f, 0.0f, 1.0f, 1.0f, 1.0f, 1.0f);
    if (rc) return rc;
    for (int m = 0; m < mask_count; ++m) {
        if (host_masks[m] < 0 || host_masks[m] >= anchor_count)
            return fail_invalid("pxh_yolo_detections: mask %d names anchor %d of %d", m, host_masks[m], anchor_count);
        p.masks[m] = host_masks[m];
    }
    for (int a = 0; a < 2 * anchor_count; ++a) p.anchors[a] = static_cast<float>(host_anchors[a]);
    const unsigned long long orders = 1ull * batch * mask_count * p.area * classes;
    if (orders + order_base > 0xFFFFFFFFull) {
        set_error("pxh_yolo_detections: emission orders past 2^32 (base %u + %llu)", order_base, orders);
        return PXH_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    DetectArgs a{};
    a.pred = predictions; a.out = out; a.count = count; a.capacity = capacity; a.threshold = threshold;
    a.image_width = image_width; a.image_height = image_height;
    a.slots = static_cast<uint32_t>(batch) * mask_count * p.area;
    a.order_base = order_base;
    a.by_area = FastDiv(p.area);
    hipLaunchKernelGGL(yolo_detect_kernel, dim3(grid_for(a.slots, kDetectBlock)), dim3(kDetectBlock), 0, s, a, p);
    return check_launch("pxh_yolo_detections");
}

int pxh_yolo_detections(const float* predictions, int batch, const int* host_masks, int mask_count,
                        const int* host_anchors, int anchor_count, int classes, int width, int height,
                        int net_width, int net_height, int image_width, int image_height, float threshold,
                        pxh_detection* out, int capacity, int* count, void* stream)
{
    if (!count) return fail_invalid("pxh_yolo_detections: null pointer");
    const int rc = pxh_fill_i32(count, 1, 0, stream);
    if (rc) return rc;
    return pxh_yolo_detections_append(predictions, batch, host_masks, mask_count, host_anchors, anchor_count, classes,
                                      width, height, net_width, net_height, image_width, image_height, threshold, 0u,
                                      out, capacity, count, stream);
}

int pxh_debug_yolo_tuning(int form, int lanes_per_slot, int head_workers)
{
    g_forced_form.store(form);
    one_launch::g_forced_lanes.store(lanes_per_slot);
    one_launch::g_forced_workers.store(head_workers);
    return 0;
}

size_t pxh_yolo_workspace_bytes(int batch, int mask_count, int classes, int width, int height, int max_truth)
{
    (void) classes;
    (void) max_truth;
    if (batch <= 0 || mask_count <= 0 || width <= 0 || height <= 0) return 0;
    return training_workspace_bytes(batch, mask_count, width, height);
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
    for (int a = 0; a < 2 * anchor_count; ++a) {
        p.anchors[a] = static_cast<float>(host_anchors[a]);
        p.anchors_rel[a] = p.anchors[a] / static_cast<float>(a % 2 ? net_height : net_width);
    }
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes, training_workspace_bytes(batch, mask_count, width, height), &ws,
                           as_stream(stream));
    if (rc) return rc;
    return run_training_pass<true>("pxh_yolo_forward_train", input, output, delta, truths, truth_counts, p,
                                   YoloTables{}, stats, cost, 0, ws, as_stream(stream));
}

static int heads_params(const char* who, int count, const pxh_yolo_head* heads, const int* host_anchors,
                        int anchor_count, int batch, int classes, int net_width, int net_height, int max_truth,
                        YoloParams* params)
{
    if (count <= 0 || count > all_heads::kMaxHeads) {
        set_error("%s: between 1 and %d heads per call, not %d", who, all_heads::kMaxHeads, count);
        return count <= 0 ? PXH_ERR_INVALID_ARGUMENT : PXH_ERR_UNSUPPORTED;
    }
    if (!heads || !host_anchors) return fail_invalid("%s: null pointer", who);
    for (int h = 0; h < count; ++h) {
        const pxh_yolo_head& hd = heads[h];
        if (!hd.input || !hd.output || !hd.delta || !hd.masks) return fail_invalid("%s: null pointer in head %d", who, h);
        if (hd.input == hd.output || hd.input == hd.delta || hd.output == hd.delta)
            return fail_invalid("%s: input, output and delta of head %d must be distinct buffers", who, h);
        YoloParams& p = params[h];
        p = YoloParams{};
        int rc = fill_params(who, p, batch, hd.mask_count, anchor_count, classes, hd.width, hd.height, net_width,
                             net_height, max_truth, hd.ignore_thresh, hd.truth_thresh, hd.coord_scale, hd.object_scale,
                             hd.noobject_scale, hd.class_scale);
        if (rc) return rc;
        for (int m = 0; m < hd.mask_count; ++m) {
            if (hd.masks[m] < 0 || hd.masks[m] >= anchor_count)
                return fail_invalid("%s: mask %d of head %d names anchor %d of %d", who, m, h, hd.masks[m], anchor_count);
            p.masks[m] = hd.masks[m];
        }
        for (int a = 0; a < 2 * anchor_count; ++a) {
            p.anchors[a] = static_cast<float>(host_anchors[a]);
            p.anchors_rel[a] = p.anchors[a] / static_cast<float>(a % 2 ? net_height : net_width);
        }
    }
    return PXH_OK;
}

size_t pxh_yolo_heads_workspace_bytes(int count, const pxh_yolo_head* heads, int batch)
{
    if (count <= 0 || count > all_heads::kMaxHeads || !heads || batch <= 0) return 0;
    for (int h = 0; h < count; ++h)
        if (heads[h].mask_count <= 0 || heads[h].width <= 0 || heads[h].height <= 0) return 0;
    return all_heads::workspace_bytes(count, heads, batch);
}

int pxh_yolo_forward_train_heads(int count, const pxh_yolo_head* heads, const float* truths, const int* truth_counts,
                                 int max_truth, const int* host_anchors, int anchor_count, int batch, int classes,
                                 int net_width, int net_height, void* workspace, size_t workspace_bytes, void* stream)
{
    const char* who = "pxh_yolo_forward_train_heads";
    if (!truth_counts || (!truths && max_truth > 0)) return fail_invalid("%s: null pointer", who);
    YoloParams params[all_heads::kMaxHeads];
    int rc = heads_params(who, count, heads, host_anchors, anchor_count, batch, classes, net_width, net_height,
                          max_truth, params);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes, all_heads::workspace_bytes(count, heads, batch), &ws,
                           as_stream(stream));
    if (rc) return rc;
    return all_heads::run(who, count, heads, params, truths, truth_counts, ws, as_stream(stream));
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
    rc = resolve_workspace(workspace, workspace_bytes, training_workspace_bytes(batch, mask_count, width, height), &ws,
                           as_stream(stream));
    if (rc) return rc;
    const YoloTables tb{ assigned_classes, assigned_anchors, assigned_boxes, masks, anchors };
    return run_training_pass<false>("pxh_yolo_loss", output, nullptr, delta, truths, truth_counts, p, tb, stats,
                                    cost, 1, ws, as_stream(stream));
}

}
