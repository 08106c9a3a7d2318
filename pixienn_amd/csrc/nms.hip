// Non-maximum suppression of detection records on the device, for gfx950.
//
// The reference runs nms (src/Box.cpp:56-147) on the host over records it copied back: a stable
// sort by probability, a pass that drops near-identical boxes of different classes, a greedy
// pass inside every (image, class) group, each of them a sequential loop.  Here the number of
// records stays on the device, so every launch is sized for the capacity and the workgroups past
// the live count leave at once.  Steps:
//   1. LSD radix sort (8-bit digits) of (probability descending, emission order) -> global rank;
//   2. two to four more stable passes on (image, class) -> groups contiguous, rank order inside;
//   3. duplicate pass as a fixed point: a record is decided once every conflicting record of
//      lower rank is; sweeps over all undecided records in parallel, states only ever move from
//      undecided to kept/dropped, so any schedule ends in the sequential loop's answer;
//   4. the greedy pass the same way, one workgroup per group, states in LDS;
//   5. compaction of the kept records in rank order.
#include "common.h"
#include "pixienn_hip_test.h"

#include <atomic>

namespace pxh {
namespace {

constexpr int kSortTile = 4096;                       // keys per workgroup and pass
constexpr int kSortRounds = kSortTile / kBlock;
constexpr int kDigits = 256;
constexpr int kWide = 1024;                           // workgroup of the single-workgroup kernels
constexpr int kGroupVisit = 1024;                     // maxCandidatesPerGroup, src/Box.cpp:105
constexpr float kDuplicateOverlap = 0.9f;             // crossClassDuplicateIoU, src/Box.cpp:71

static_assert(kDigits == kBlock, "one bin per lane of the sorting workgroups");

enum : uint32_t { kUndecided = 0, kKept = 1, kDropped = 2, kAbsent = 3 };

__device__ __forceinline__ uint32_t live_count(const int* count, int capacity)
{
    const int n = *count;
    return n < 0 ? 0u : static_cast<uint32_t>(n > capacity ? capacity : n);
}

// States are written by one lane and read by lanes of other workgroups while a kernel runs:
// both sides go to the device-coherent level.
__device__ __forceinline__ uint32_t load_state(const uint32_t* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_state(uint32_t* p, uint32_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Exclusive prefix sum of one value per lane over a kWide-lane workgroup; `total` in every lane.
__device__ __forceinline__ uint32_t wide_exclusive_scan(uint32_t v, uint32_t* lds /* kWide / kWave + 1 */,
                                                        uint32_t& total)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += up;
    }
    __syncthreads();
    if (lane == kWave - 1) lds[wave] = incl;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (int w = 0; w < kWide / kWave; ++w) {
            const uint32_t t = lds[w];
            lds[w] = run;
            run += t;
        }
        lds[kWide / kWave] = run;
    }
    __syncthreads();
    total = lds[kWide / kWave];
    return lds[wave] + incl - v;
}

// ---------------------------------------------------------------- radix sort passes
struct SortArgs {
    const uint64_t* keys_in;
    const uint32_t* vals_in;
    uint64_t* keys_out;
    uint32_t* vals_out;
    uint32_t* hist;          // [digit][live tiles]
    const int* count;
    int capacity;
    int shift;
};

__device__ __forceinline__ uint32_t live_tiles(uint32_t n) { return (n + kSortTile - 1) / kSortTile; }

__global__ __launch_bounds__(kBlock) void sort_histogram_kernel(SortArgs a)
{
    __shared__ uint32_t bins[kDigits];
    const uint32_t n = live_count(a.count, a.capacity);
    const uint32_t tiles = live_tiles(n);
    if (blockIdx.x >= tiles) return;
    bins[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t first = blockIdx.x * kSortTile;
    for (int r = 0; r < kSortRounds; ++r) {
        const uint32_t i = first + r * kBlock + threadIdx.x;
        if (i < n) atomicAdd(&bins[(a.keys_in[i] >> a.shift) & (kDigits - 1)], 1u);
    }
    __syncthreads();
    a.hist[threadIdx.x * tiles + blockIdx.x] = bins[threadIdx.x];
}

// In-place exclusive prefix sum over `per_tile` * (live tiles) counters by ONE workgroup; the sum of
// all of them goes to *total_out when given.
__global__ __launch_bounds__(kWide) void scan_counters_kernel(uint32_t* counters, const int* count, int capacity,
                                                              uint32_t per_tile, int* total_out)
{
    __shared__ uint32_t lds[kWide / kWave + 1];
    const uint32_t n = live_count(count, capacity);
    const uint32_t entries = per_tile * live_tiles(n);
    const uint32_t per = (entries + kWide - 1) / kWide;
    const uint32_t lo = min(threadIdx.x * per, entries);
    const uint32_t hi = min(lo + per, entries);
    uint32_t sum = 0;
    for (uint32_t i = lo; i < hi; ++i) sum += counters[i];
    uint32_t total;
    uint32_t run = wide_exclusive_scan(sum, lds, total);
    for (uint32_t i = lo; i < hi; ++i) {
        const uint32_t c = counters[i];
        counters[i] = run;
        run += c;
    }
    if (total_out && threadIdx.x == 0) *total_out = static_cast<int>(total);
}

__global__ __launch_bounds__(kBlock) void sort_scatter_kernel(SortArgs a)
{
    __shared__ uint32_t base[kDigits];
    __shared__ uint32_t wave_count[kBlock / kWave][kDigits];
    const uint32_t n = live_count(a.count, a.capacity);
    const uint32_t tiles = live_tiles(n);
    if (blockIdx.x >= tiles) return;
    base[threadIdx.x] = a.hist[threadIdx.x * tiles + blockIdx.x];
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) wave_count[w][threadIdx.x] = 0;
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
    const uint32_t first = blockIdx.x * kSortTile;
    for (int r = 0; r < kSortRounds; ++r) {
        if (first + r * kBlock >= n) break;                               // the same for every lane
        const uint32_t i = first + r * kBlock + threadIdx.x;
        const bool valid = i < n;
        const uint64_t key = valid ? a.keys_in[i] : 0ull;
        const uint32_t val = valid ? a.vals_in[i] : 0u;
        const uint32_t digit = static_cast<uint32_t>(key >> a.shift) & (kDigits - 1);
        // lanes of this wave that hold the same digit
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            const bool set = (digit >> bit) & 1u;
            const uint64_t with = __ballot(set);
            peers &= set ? with : ~with;
        }
        const uint32_t rank = __popcll(peers & below);
        if (valid && rank == 0) wave_count[wave][digit] = __popcll(peers);
        __syncthreads();
        if (valid) {
            uint32_t at = base[digit] + rank;
            for (int w = 0; w < wave; ++w) at += wave_count[w][digit];
            a.keys_out[at] = key;
            a.vals_out[at] = val;
        }
        __syncthreads();
        uint32_t add = 0;
#pragma unroll
        for (int w = 0; w < kBlock / kWave; ++w) {
            add += wave_count[w][threadIdx.x];
            wave_count[w][threadIdx.x] = 0;
        }
        base[threadIdx.x] += add;
        __syncthreads();
    }
}

// ---------------------------------------------------------------- keys
// Ascending key order = descending probability, then ascending emission order.
__device__ __forceinline__ uint32_t descending_bits(float v)
{
    const uint32_t u = __float_as_uint(v);
    const uint32_t ascending = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ~ascending;
}

__global__ __launch_bounds__(kBlock) void nms_rank_keys_kernel(const pxh_detection* records, const int* count,
                                                               int capacity, uint64_t* keys, uint32_t* vals,
                                                               uint32_t* counters)
{
    const uint32_t n = live_count(count, capacity);
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (blockIdx.x == 0 && threadIdx.x < 8) counters[threadIdx.x] = 0;
    if (i >= n) return;
    const pxh_detection d = records[i];
    keys[i] = (static_cast<uint64_t>(descending_bits(d.prob)) << 32) | d.order;
    vals[i] = i;
}

// sorted[r] = input index of the record of rank r  ->  perm, and the keys of the second sort
// An image or class number outside [0, batch) x [0, classes) is clamped into it for the grouping,
// so that the groups stay contiguous whatever the records hold.
__global__ __launch_bounds__(kBlock) void nms_group_keys_kernel(const pxh_detection* records, const int* count,
                                                                int capacity, const uint32_t* sorted, uint32_t* perm,
                                                                uint64_t* keys, uint32_t* vals, int batch, int classes)
{
    const uint32_t n = live_count(count, capacity);
    const uint32_t r = blockIdx.x * kBlock + threadIdx.x;
    if (r >= n) return;
    const uint32_t at = sorted[r];
    perm[r] = at;
    const pxh_detection d = records[at];
    const uint32_t image = static_cast<uint32_t>(min(max(d.batch, 0), batch - 1));
    const uint32_t cls = static_cast<uint32_t>(min(max(d.class_index, 0), classes - 1));
    keys[r] = (static_cast<uint64_t>(image) << 32) | cls;
    vals[r] = r;
}

__device__ __forceinline__ uint32_t lower_bound(const uint64_t* keys, uint32_t n, uint64_t key)
{
    uint32_t lo = 0, hi = n;
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2;
        if (keys[mid] < key) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

// ---------------------------------------------------------------- boxes
// normalizedRect, src/Box.cpp:47-54: (x1, y1, w, h)
__device__ __forceinline__ float4 normalized_rect(const pxh_detection& d)
{
    const float xe = d.x + d.w, ye = d.y + d.h;
    const float x1 = fminf(d.x, xe), y1 = fminf(d.y, ye);
    const float x2 = fmaxf(d.x, xe), y2 = fmaxf(d.y, ye);
    return make_float4(x1, y1, fmaxf(0.0f, x2 - x1), fmaxf(0.0f, y2 - y1));
}

// boxIoU(a, b) > threshold, src/Box.cpp:25-45, with cv::Rect2f's operator& (OpenCV >= 4.5.4): an
// empty operand or a non-positive extent gives no overlap; the extent along an axis is
// min(lo.size - (hi.origin - lo.origin), hi.size) with lo/hi ordered by origin.  threshold >= 0, so
// no overlap can never be above it; and the union is at least the larger area, so an overlap well
// below threshold * that area is decided without the division (the margin of a tenth is far more
// than all rounding involved).  Everything else takes the reference's own operations.
__device__ __forceinline__ bool overlaps_above(const float4 a, const float4 b, float threshold)
{
    if (a.z <= 0.0f || a.w <= 0.0f || b.z <= 0.0f || b.w <= 0.0f) return false;
    const bool ax = a.x < b.x, ay = a.y < b.y;
    const float xlo = ax ? a.x : b.x, xlo_w = ax ? a.z : b.z, xhi = ax ? b.x : a.x, xhi_w = ax ? b.z : a.z;
    const float ylo = ay ? a.y : b.y, ylo_h = ay ? a.w : b.w, yhi = ay ? b.y : a.y, yhi_h = ay ? b.w : a.w;
    if ((xlo < 0.0f && xlo + xlo_w < xhi) || (ylo < 0.0f && ylo + ylo_h < yhi)) return false;
    const float iw = fminf(xlo_w - (xhi - xlo), xhi_w);
    const float ih = fminf(ylo_h - (yhi - ylo), yhi_h);
    if (!(iw > 0.0f && ih > 0.0f)) return false;
    const float inter = iw * ih;
    const float area_a = a.z * a.w, area_b = b.z * b.w;
    if (inter < 0.9f * threshold * fmaxf(area_a, area_b)) return false;
    float uni = area_a + area_b - inter;
    if (!(0.0f < uni)) uni = 0.0f;
    const float q = inter / uni;
    if (isnan(q) || isinf(q)) return false;          // counts as no overlap: 0 > threshold is false
    return q > threshold;
}

struct Segments {
    uint32_t image_begin, image_end, group_begin, group_end;
};

struct NmsArgs {
    const pxh_detection* records;
    const int* count;
    int capacity;
    const uint32_t* perm;      // rank -> input index
    const uint64_t* group_key; // per place (sorted by image, class, rank)
    const uint32_t* rank;      // per place
    float4* box;               // per place
    Segments* seg;             // per place
    uint32_t* state;           // per place, duplicate pass
    uint32_t* keep;            // per rank
    uint32_t* resume;          // per place: where the next sweep of the duplicate pass continues
    uint32_t* counters;        // [k] != 0: sweep k left records undecided
    uint32_t waves;            // waves of a duplicate sweep's grid
};

__global__ __launch_bounds__(kBlock) void nms_gather_kernel(NmsArgs a)
{
    const uint32_t n = live_count(a.count, a.capacity);
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    a.box[p] = normalized_rect(a.records[a.perm[a.rank[p]]]);
    const uint64_t key = a.group_key[p];
    const uint64_t image = key & 0xFFFFFFFF00000000ull;
    Segments s;
    s.image_begin = lower_bound(a.group_key, n, image);
    s.image_end = lower_bound(a.group_key, n, image + 0x100000000ull);
    s.group_begin = lower_bound(a.group_key, n, key);
    s.group_end = lower_bound(a.group_key, n, key + 1ull);
    a.seg[p] = s;
    a.state[p] = kUndecided;
    a.resume[p] = s.image_begin;
}

// ---------------------------------------------------------------- duplicate pass
// src/Box.cpp:65-88: a record is dropped when an earlier KEPT record of the same image and another
// class overlaps it by more than 0.9.  One WAVE per undecided record, its lanes side by side over
// the other places of the image (the record's own class group is stepped over).  Outcome for the
// record at place p: 1 = dropped, 0 = kept, 2 = still waiting for an undecided earlier record, in
// which case resume[p] is the first such place: everything before it that conflicts is dropped for
// good and need not be looked at again.
__device__ __forceinline__ int duplicate_scan(const NmsArgs& a, uint32_t p, int lane)
{
    const Segments s = a.seg[p];
    const float4 box = a.box[p];
    const uint32_t rank = a.rank[p];
    uint32_t first_pending = 0xFFFFFFFFu;
    uint32_t q0 = a.resume[p];
    while (q0 < s.image_end) {
        if (q0 >= s.group_begin && q0 < s.group_end) {          // the same class: not compared
            q0 = s.group_end;
            continue;
        }
        const uint32_t stop = q0 < s.group_begin ? s.group_begin : s.image_end;
        const uint32_t q = q0 + lane;
        bool kept_hit = false, waiting = false;
        if (q < stop && a.rank[q] < rank) {
            const uint32_t st = load_state(a.state + q);
            if (st != kDropped && overlaps_above(box, a.box[q], kDuplicateOverlap)) {
                kept_hit = st == kKept;
                waiting = st == kUndecided;
            }
        }
        if (__ballot(kept_hit)) return 1;
        const uint64_t w = __ballot(waiting);
        if (w && first_pending == 0xFFFFFFFFu) first_pending = q0 + __builtin_ctzll(w);
        q0 = min(q0 + kWave, stop);
    }
    if (first_pending == 0xFFFFFFFFu) return 0;
    if (lane == 0) a.resume[p] = first_pending;
    return 2;
}

__global__ __launch_bounds__(kBlock) void nms_duplicate_sweep_kernel(NmsArgs a, int sweep)
{
    const uint32_t n = live_count(a.count, a.capacity);
    if (sweep > 0 && a.counters[sweep - 1] == 0) return;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) / kWave;
    bool left = false;
    for (uint32_t p = wave; p < n; p += a.waves) {
        if (load_state(a.state + p) != kUndecided) continue;
        const int outcome = duplicate_scan(a, p, lane);
        if (outcome == 2) left = true;
        else if (lane == 0) store_state(a.state + p, outcome == 1 ? kDropped : kKept);
    }
    if (left && lane == 0) store_state(a.counters + sweep, 1u);
}

// What the sweeps left undecided (long chains of conflicts): one workgroup per image repeats the
// sweep over its own records until none is left.  Every repetition decides at least the undecided
// record of lowest rank, so the loop ends.
__global__ __launch_bounds__(kWide) void nms_duplicate_finish_kernel(NmsArgs a, int last_sweep)
{
    if (a.counters[last_sweep] == 0) return;
    const uint32_t n = live_count(a.count, a.capacity);
    const uint64_t image = static_cast<uint64_t>(blockIdx.x) << 32;
    const uint32_t begin = lower_bound(a.group_key, n, image);
    const uint32_t end = lower_bound(a.group_key, n, image + 0x100000000ull);
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    // one repetition per record is the most the argument above allows; the bound makes the exit
    // unconditional
    for (uint32_t repetition = 0; repetition <= end - begin; ++repetition) {
        int left = 0;
        for (uint32_t p = begin + wave; p < end; p += kWide / kWave) {
            if (load_state(a.state + p) != kUndecided) continue;
            const int outcome = duplicate_scan(a, p, lane);
            if (outcome == 2) left = 1;
            else if (lane == 0) store_state(a.state + p, outcome == 1 ? kDropped : kKept);
        }
        __threadfence();
        if (__syncthreads_or(left) == 0) break;
    }
}

// ---------------------------------------------------------------- greedy pass inside a group
// src/Box.cpp:104-136: the first 1024 places of the group in rank order; a record the duplicate
// pass dropped is skipped; a record is suppressed when an earlier KEPT one overlaps it by more than
// the threshold.  One workgroup per (image, class), one lane per place, states in LDS.
__global__ __launch_bounds__(kWide) void nms_group_kernel(NmsArgs a, float threshold, FastDiv by_classes)
{
    __shared__ float4 group_box[kGroupVisit];
    __shared__ uint32_t group_state[kGroupVisit];
    const uint32_t n = live_count(a.count, a.capacity);
    if (n == 0) return;
    uint32_t image, cls;
    by_classes.divmod(blockIdx.x, image, cls);
    const uint64_t key = (static_cast<uint64_t>(image) << 32) | cls;
    const uint32_t begin = lower_bound(a.group_key, n, key);
    const uint32_t end = lower_bound(a.group_key, n, key + 1ull);
    if (begin == end) return;
    const uint32_t visit = min(end - begin, static_cast<uint32_t>(kGroupVisit));
    const uint32_t t = threadIdx.x;
    const bool active = t < visit;
    float4 box = make_float4(0, 0, 0, 0);
    bool decided = true;
    if (active) {
        box = a.box[begin + t];
        const bool alive = load_state(a.state + begin + t) == kKept;
        group_box[t] = box;
        group_state[t] = alive ? kUndecided : kAbsent;
        decided = !alive;
    }
    __syncthreads();
    const volatile uint32_t* states = group_state;
    uint32_t from = 0;
    // each repetition decides at least the undecided place of lowest rank: at most `visit` of them
    for (uint32_t repetition = 0; repetition <= visit; ++repetition) {
        if (!decided) {
            bool drop = false, pending = false;
            uint32_t first_pending = t;
            for (uint32_t j = from; j < t; ++j) {
                const uint32_t st = states[j];
                if (st == kAbsent || st == kDropped) continue;
                if (overlaps_above(box, group_box[j], threshold)) {
                    if (st == kKept) {
                        drop = true;
                        break;
                    }
                    if (!pending) {
                        pending = true;
                        first_pending = j;
                    }
                }
            }
            if (drop) {
                group_state[t] = kDropped;
                decided = true;
            } else if (!pending) {
                group_state[t] = kKept;
                decided = true;
            } else {
                from = first_pending;      // everything before it that overlaps is dropped for good
            }
        }
        if (__syncthreads_count(!decided) == 0) break;
    }
    if (active) a.keep[a.rank[begin + t]] = group_state[t] == kKept ? 1u : 0u;
    // places past the first 1024 are never visited: they stay unless the duplicate pass dropped them
    for (uint32_t p = begin + kGroupVisit + t; p < end; p += kWide)
        a.keep[a.rank[p]] = load_state(a.state + p) == kKept ? 1u : 0u;
}

// ---------------------------------------------------------------- compaction in rank order
__global__ __launch_bounds__(kBlock) void nms_count_kept_kernel(NmsArgs a, uint32_t* tile_kept)
{
    __shared__ uint32_t sum;
    const uint32_t n = live_count(a.count, a.capacity);
    if (blockIdx.x >= live_tiles(n)) return;
    if (threadIdx.x == 0) sum = 0;
    __syncthreads();
    uint32_t mine = 0;
    const uint32_t first = blockIdx.x * kSortTile;
    for (int r = 0; r < kSortRounds; ++r) {
        const uint32_t i = first + r * kBlock + threadIdx.x;
        if (i < n) mine += a.keep[i];
    }
    if (mine) atomicAdd(&sum, mine);
    __syncthreads();
    if (threadIdx.x == 0) tile_kept[blockIdx.x] = sum;
}

__global__ __launch_bounds__(kBlock) void nms_write_kept_kernel(NmsArgs a, const uint32_t* tile_first,
                                                                pxh_detection* kept)
{
    __shared__ uint32_t wave_kept[kBlock / kWave];
    const uint32_t n = live_count(a.count, a.capacity);
    if (blockIdx.x >= live_tiles(n)) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint64_t below = (1ull << lane) - 1ull;
    uint32_t base = tile_first[blockIdx.x];
    const uint32_t first = blockIdx.x * kSortTile;
    for (int r = 0; r < kSortRounds; ++r) {
        if (first + r * kBlock >= n) break;                               // the same for every lane
        const uint32_t i = first + r * kBlock + threadIdx.x;
        const bool take = i < n && a.keep[i] != 0;
        const uint64_t takers = __ballot(take);
        if (lane == 0) wave_kept[wave] = __popcll(takers);
        __syncthreads();
        uint32_t at = base + __popcll(takers & below);
        uint32_t all = 0;
#pragma unroll
        for (int w = 0; w < kBlock / kWave; ++w) {
            const uint32_t c = wave_kept[w];
            if (w < wave) at += c;
            all += c;
        }
        if (take) kept[at] = a.records[a.perm[i]];
        base += all;
        __syncthreads();
    }
}

// ---------------------------------------------------------------- short lists in one workgroup
// Up to 512 records (what an inference pass leaves): everything above in ONE launch, with the
// records in LDS.  Ranks come from counting the smaller keys.  Both passes take one wave per record,
// lanes side by side over the records of lower rank, and the waves walk the ranks in ascending
// order, so nearly every record finds the ones it depends on already decided; the few that do not
// are taken again.  No group can reach the 1024-place limit.
constexpr int kSmall = 512;

// One pass over the ranks: `same_class` false = duplicates across classes (src/Box.cpp:65-88), true =
// greedy suppression inside (image, class) (src/Box.cpp:104-136).
__device__ __forceinline__ void small_pass(uint32_t n, bool same_class, float threshold, const float4* ranked_box,
                                           const uint2* ranked_group, uint32_t* state)
{
    const volatile uint32_t* states = state;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    // a repetition decides at least the undecided record of lowest rank; the bound makes the exit
    // unconditional
    for (uint32_t repetition = 0; repetition <= n; ++repetition) {
        int left = 0;
        for (uint32_t t = wave; t < n; t += kWide / kWave) {
            if (states[t] != kUndecided) continue;
            const float4 box = ranked_box[t];
            const uint2 group = ranked_group[t];
            bool drop = false, pending = false;
            for (uint32_t j0 = 0; j0 < t && !drop; j0 += kWave) {
                const uint32_t j = j0 + lane;
                bool hit = false, wait = false;
                if (j < t) {
                    const uint2 other = ranked_group[j];
                    if (other.x == group.x && (other.y == group.y) == same_class) {
                        const uint32_t st = states[j];
                        if ((st == kKept || st == kUndecided) && overlaps_above(box, ranked_box[j], threshold)) {
                            hit = st == kKept;
                            wait = st == kUndecided;
                        }
                    }
                }
                drop = __ballot(hit) != 0;
                pending = pending || __ballot(wait) != 0;
            }
            if (drop || !pending) {
                if (lane == 0) state[t] = drop ? kDropped : kKept;
            } else {
                left = 1;
            }
        }
        if (__syncthreads_or(left) == 0) break;
    }
}

__global__ __launch_bounds__(kWide) void nms_small_kernel(const pxh_detection* records, const int* count, int capacity,
                                                          int batch, int classes, float threshold,
                                                          pxh_detection* kept, int* kept_count)
{
    __shared__ uint64_t key[kSmall];
    __shared__ float4 ranked_box[kSmall];
    __shared__ uint2 ranked_group[kSmall];       // image, class
    __shared__ uint32_t source[kSmall];
    __shared__ uint32_t state[kSmall];
    __shared__ uint32_t scan_lds[kWide / kWave + 1];
    const uint32_t n = live_count(count, capacity);
    const uint32_t t = threadIdx.x;
    const bool valid = t < n;
    pxh_detection d{};
    if (valid) {
        d = records[t];
        key[t] = (static_cast<uint64_t>(descending_bits(d.prob)) << 32) | d.order;
    }
    __syncthreads();
    if (valid) {
        const uint64_t mine = key[t];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < n; ++j) {
            const uint64_t k = key[j];
            rank += (k < mine || (k == mine && j < t)) ? 1u : 0u;
        }
        ranked_box[rank] = normalized_rect(d);
        ranked_group[rank] = make_uint2(static_cast<uint32_t>(min(max(d.batch, 0), batch - 1)),
                                        static_cast<uint32_t>(min(max(d.class_index, 0), classes - 1)));
        source[rank] = t;
        state[rank] = kUndecided;
    }
    __syncthreads();
    small_pass(n, false, kDuplicateOverlap, ranked_box, ranked_group, state);
    // survivors of the first pass enter the second; the dropped ones are absent from it
    if (valid) state[t] = state[t] == kKept ? kUndecided : kAbsent;
    __syncthreads();
    small_pass(n, true, threshold, ranked_box, ranked_group, state);
    const bool take = valid && state[t] == kKept;
    uint32_t total;
    const uint32_t at = wide_exclusive_scan(take ? 1u : 0u, scan_lds, total);
    if (take) kept[at] = records[source[t]];
    if (t == 0) *kept_count = static_cast<int>(total);
}

size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }

struct Workspace {
    uint64_t* keys[2];
    uint32_t* vals[2];
    uint32_t* perm;
    float4* box;
    Segments* seg;
    uint32_t* state;
    uint32_t* keep;
    uint32_t* resume;
    uint32_t* hist;
    uint32_t* tile_kept;
    uint32_t* counters;
    size_t bytes;
};

Workspace carve(void* base, int capacity)
{
    const size_t cap = static_cast<size_t>(capacity > 0 ? capacity : 1);
    const size_t tiles = (cap + kSortTile - 1) / kSortTile;
    char* p = static_cast<char*>(base);
    size_t at = 0;
    auto take = [&](size_t bytes) {
        char* r = p ? p + at : nullptr;
        at += align256(bytes);
        return r;
    };
    Workspace w{};
    w.keys[0] = reinterpret_cast<uint64_t*>(take(cap * 8));
    w.keys[1] = reinterpret_cast<uint64_t*>(take(cap * 8));
    w.vals[0] = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.vals[1] = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.perm = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.box = reinterpret_cast<float4*>(take(cap * 16));
    w.seg = reinterpret_cast<Segments*>(take(cap * sizeof(Segments)));
    w.state = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.keep = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.resume = reinterpret_cast<uint32_t*>(take(cap * 4));
    w.hist = reinterpret_cast<uint32_t*>(take(tiles * kDigits * 4));
    w.tile_kept = reinterpret_cast<uint32_t*>(take(tiles * 4));
    w.counters = reinterpret_cast<uint32_t*>(take(8 * 4));
    w.bytes = at;
    return w;
}

std::atomic<int> g_sweeps{ 6 };      // parallel sweeps of the duplicate pass before the per-image loop takes over

}  // namespace
}  // namespace pxh

using namespace pxh;

extern "C" {

size_t pxh_nms_workspace_bytes(int capacity)
{
    if (capacity <= 0) return 0;
    return carve(nullptr, capacity).bytes;
}

int pxh_debug_nms_sweeps(int sweeps)
{
    if (sweeps >= 1 && sweeps <= 6) return g_sweeps.exchange(sweeps);
    return g_sweeps.load();
}

int pxh_nms(const pxh_detection* records, const int* count, int capacity, int batch, int classes, float threshold,
            pxh_detection* kept, int* kept_count, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!count || !kept_count || (capacity > 0 && (!records || !kept))) return fail_invalid("pxh_nms: null pointer");
    if (capacity < 0 || batch <= 0 || classes <= 0)
        return fail_invalid("pxh_nms: capacity must not be negative, batch and classes must be positive");
    if (!(threshold >= 0.0f)) return fail_invalid("pxh_nms: the threshold must not be negative");
    if (1ull * batch * classes >= (1ull << 31)) {
        set_error("pxh_nms: batch * classes of 2^31 or more is not supported");
        return PXH_ERR_UNSUPPORTED;
    }
    if (records == kept && capacity > 0) return fail_invalid("pxh_nms: records and kept must be distinct buffers");
    if (capacity == 0) return pxh_fill_i32(kept_count, 1, 0, stream);
    if (capacity <= kSmall) {
        hipLaunchKernelGGL(nms_small_kernel, dim3(1), dim3(kWide), 0, as_stream(stream), records, count, capacity,
                           batch, classes, threshold, kept, kept_count);
        return check_launch("pxh_nms");
    }
    void* ws;
    int rc = resolve_workspace(workspace, workspace_bytes, carve(nullptr, capacity).bytes, &ws, as_stream(stream));
    if (rc) return rc;
    const Workspace w = carve(ws, capacity);
    hipStream_t s = as_stream(stream);
    const dim3 per_record(grid_for(capacity, kBlock)), per_tile(grid_for(capacity, kSortTile));
    const dim3 lanes(kBlock), wide(kWide);

    hipLaunchKernelGGL(nms_rank_keys_kernel, per_record, lanes, 0, s, records, count, capacity, w.keys[0], w.vals[0],
                       w.counters);
    int from = 0;
    auto sort_pass = [&](int shift) {
        SortArgs a{ w.keys[from], w.vals[from], w.keys[1 - from], w.vals[1 - from], w.hist, count, capacity, shift };
        hipLaunchKernelGGL(sort_histogram_kernel, per_tile, lanes, 0, s, a);
        hipLaunchKernelGGL(scan_counters_kernel, dim3(1), wide, 0, s, w.hist, count, capacity,
                           static_cast<uint32_t>(kDigits), static_cast<int*>(nullptr));
        hipLaunchKernelGGL(sort_scatter_kernel, per_tile, lanes, 0, s, a);
        from = 1 - from;
    };
    for (int shift = 0; shift < 64; shift += 8) sort_pass(shift);
    // keys of the second sort go to the other buffer pair; vals[from] still holds rank -> input index
    hipLaunchKernelGGL(nms_group_keys_kernel, per_record, lanes, 0, s, records, count, capacity, w.vals[from], w.perm,
                       w.keys[1 - from], w.vals[1 - from], batch, classes);
    from = 1 - from;
    for (int shift = 0; ((classes - 1) >> shift) > 0; shift += 8) sort_pass(shift);
    for (int shift = 0; ((batch - 1) >> shift) > 0; shift += 8) sort_pass(32 + shift);

    NmsArgs a{};
    a.records = records; a.count = count; a.capacity = capacity; a.perm = w.perm;
    a.group_key = w.keys[from]; a.rank = w.vals[from];
    a.box = w.box; a.seg = w.seg; a.state = w.state; a.keep = w.keep; a.resume = w.resume; a.counters = w.counters;
    hipLaunchKernelGGL(nms_gather_kernel, per_record, lanes, 0, s, a);
    const int sweeps = g_sweeps.load();      // read once: a call never sees it change
    // one wave per record, at most 64 Ki workgroups (the rest of a longer list comes round again)
    const unsigned sweep_blocks = grid_for(capacity, kBlock / kWave) < 65536u ? grid_for(capacity, kBlock / kWave) : 65536u;
    a.waves = sweep_blocks * (kBlock / kWave);
    for (int k = 0; k < sweeps; ++k)
        hipLaunchKernelGGL(nms_duplicate_sweep_kernel, dim3(sweep_blocks), lanes, 0, s, a, k);
    hipLaunchKernelGGL(nms_duplicate_finish_kernel, dim3(batch), wide, 0, s, a, sweeps - 1);
    hipLaunchKernelGGL(nms_group_kernel, dim3(static_cast<unsigned>(batch) * classes), wide, 0, s, a, threshold,
                       FastDiv(classes));
    hipLaunchKernelGGL(nms_count_kept_kernel, per_tile, lanes, 0, s, a, w.tile_kept);
    hipLaunchKernelGGL(scan_counters_kernel, dim3(1), wide, 0, s, w.tile_kept, count, capacity, 1u, kept_count);
    hipLaunchKernelGGL(nms_write_kept_kernel, per_tile, lanes, 0, s, a, w.tile_kept, kept);
    return check_launch("pxh_nms");
}

}
