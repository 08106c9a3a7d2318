// Conv-layer epilogue for gfx950: batch-norm (inference and training) + bias + activation,
// forward and backward, as one-pass NCHW streaming kernels and per-channel reductions.
//
// Numerics follow the CPU layer (src/BatchNorm.cpp, src/CpuUtil.cpp:248-342 of the reference):
//   x_hat = float( double(x - mean) / (sqrt(double(var)) + 1e-5f) )     eps OUTSIDE the root
//   pre   = float(float(x_hat * scale) + bias)                           two fp32 roundings
// The per-channel reciprocal R = 1 / (sqrt(double(var)) + eps) is formed once per channel in
// fp64 and kept as two floats (hi + lo); x_hat = fma(t, hi, t * lo) then rounds t * R once, which
// equals the rounded double quotient except in about 1e-7 of the elements (1 ulp there).
#include "stream.h"

#include <mutex>
#include <vector>

// Device memory for pxh_bn_train_act_forward_static, the entry point for callers that must not
// allocate: the partial sums and per-channel constants its kernels pass from one launch to the next.
// Every GPU the library runs on holds its own copy until the process ends.  In host code the name is
// only a handle for hipGetSymbolAddress; kernels are given the address that call returns.
constexpr size_t kStaticScratchBytes = PXH_BN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace pxh {
namespace {

constexpr float kEps = .00001f;

// The device address of `scratch` on the current device, looked up once per device.
int static_scratch(const char* who, void** out)
{
    constexpr int kDevices = 64;
    static std::mutex mutex;
    static void* address[kDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        set_error("%s: hipGetDevice: %s", who, hipGetErrorString(e));
        return static_cast<int>(e);
    }
    if (dev < 0 || dev >= kDevices) {
        set_error("%s: device %d is beyond the %d devices the library keeps scratch addresses for", who, dev,
                  kDevices);
        return PXH_ERR_UNSUPPORTED;
    }
    std::lock_guard<std::mutex> lock(mutex);
    if (!address[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
            return e != hipSuccess ? static_cast<int>(e) : PXH_ERR_WORKSPACE;
        }
        address[dev] = p;
    }
    *out = address[dev];
    return PXH_OK;
}

// Folded per-channel constants of the forward pass (32 bytes: two 128-bit loads).
struct __attribute__((aligned(16))) FoldCoef {
    float mean, r_hi, r_lo, scale;
    float bias, pad0, pad1, pad2;
};

__device__ __forceinline__ FoldCoef make_coef(float mean, float var, float scale, float bias)
{
    const double r = 1.0 / (sqrt(static_cast<double>(var)) + static_cast<double>(kEps));
    FoldCoef k;
    k.mean = mean;
    k.r_hi = static_cast<float>(r);
    k.r_lo = static_cast<float>(r - static_cast<double>(k.r_hi));
    k.scale = scale;
    k.bias = bias;
    k.pad0 = k.pad1 = k.pad2 = 0.0f;
    return k;
}

__device__ __forceinline__ float normalize(float x, const FoldCoef& k)
{
    const float t = x - k.mean;
    return fmaf(t, k.r_hi, t * k.r_lo);
}

// pre-activation from x_hat: scale then bias, each rounded
__device__ __forceinline__ float affine(float xn, const FoldCoef& k)
{
    const float s = xn * k.scale;
    return s + k.bias;
}

__global__ __launch_bounds__(kBlock) void bn_fold_kernel(const float* mean, const float* var, const float* scale,
                                                         const float* bias, int channels, FoldCoef* table)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c < channels) table[c] = make_coef(mean[c], var[c], scale[c], bias[c]);
}

struct EpilogueArgs {
    const float* x;
    float* y;
    float* pre;        // nullable
    float* x_saved;    // nullable
    float* x_norm;     // nullable
    const FoldCoef* table;   // BN
    const float* bias;       // bias only
    FastDiv by_spatial;
    FastDiv by_channels;
    uint32_t total;
    // the shortcut that follows the layer, taken into the same pass (else null): what is stored in y is
    // res_alpha * act(pre) + res_beta * residual, the two products and the sum each rounded
    const float* residual;
    float res_alpha, res_beta;
};

// The linear shortcut on top of an activation's result (cuda/ShortcutLayer.h:23-37 with a linear
// activation: alpha * input + beta * from).
__device__ __forceinline__ float with_residual(float y, float from, float alpha, float beta)
{
    const float pa = alpha * y;
    const float pb = beta * from;
    return pa + pb;
}

template<bool BN>
__device__ __forceinline__ FoldCoef fetch_coef(const EpilogueArgs& a, uint32_t c)
{
    if constexpr (BN) {
        return a.table[c];
    } else {
        FoldCoef k;
        k.bias = a.bias[c];
        return k;
    }
}

template<bool BN>
__device__ __forceinline__ float pre_value(float x, const FoldCoef& k, float& xn)
{
    if constexpr (BN) {
        xn = normalize(x, k);
        return affine(xn, k);
    } else {
        xn = 0.0f;
        return x + k.bias;
    }
}

// One 128-bit vector per lane over the flat tensor.  A lane finds its plane with one
// multiply-high division and loads that channel's folded constants (a 32-byte, cache-resident
// broadcast); the rare vector that straddles two planes loads the next channel's as well.
template<int ACT, bool BN, bool NT, bool RES>
__device__ __forceinline__ void epilogue_fwd_body(const EpilogueArgs& a)
{
    const uint32_t e = (blockIdx.x * static_cast<uint32_t>(kBlock) + threadIdx.x) * 4;
    if (e >= a.total) return;
    const bool full = e + 3 < a.total;
    Pack<4> xin;
    [[maybe_unused]] Pack<4> rin;
    if (full) {
        xin = ld<4, NT>(a.x, e);
        if constexpr (RES) rin = ld<4, NT>(a.residual, e);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            xin.v[k] = (e + k < a.total) ? a.x[e + k] : 0.0f;
            if constexpr (RES) rin.v[k] = (e + k < a.total) ? a.residual[e + k] : 0.0f;
        }
    }
    const uint32_t hw = a.by_spatial.d;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    const FoldCoef k0 = fetch_coef<BN>(a, c);
    Pack<4> yo, po, no;
    const bool crosses = !(r + 3 < hw);
    if (!__ballot(crosses)) {
        // no lane of the wave touches a plane boundary (the common case for large planes)
#pragma unroll
        for (int j = 0; j < 4; ++j) po.v[j] = pre_value<BN>(xin.v[j], k0, no.v[j]);
        act_apply_n<ACT>(po.v, yo.v);
    } else if (hw >= 4) {
        // some lane's vector runs into the next plane (at most one boundary per vector): the
        // elements past it take the next channel's constants.  Selecting the constants per element
        // keeps ONE copy of the arithmetic for the whole wave; a per-lane branch would make a wave
        // that holds a boundary (every wave, for a 13 x 13 plane) run the activation twice.
        FoldCoef k1 = k0;
        if (crosses) k1 = fetch_coef<BN>(a, c + 1 == a.by_channels.d ? 0 : c + 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool here = r + j < hw;
            FoldCoef k;
            k.mean = here ? k0.mean : k1.mean;
            k.r_hi = here ? k0.r_hi : k1.r_hi;
            k.r_lo = here ? k0.r_lo : k1.r_lo;
            k.scale = here ? k0.scale : k1.scale;
            k.bias = here ? k0.bias : k1.bias;
            po.v[j] = pre_value<BN>(xin.v[j], k, no.v[j]);
        }
        act_apply_n<ACT>(po.v, yo.v);
    } else {
        // planes of fewer than 4 elements: several boundaries per vector, walk element by element
        FoldCoef k = k0;
        uint32_t rr = r, cc = c;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (rr == hw) {
                rr = 0;
                cc = cc + 1 == a.by_channels.d ? 0 : cc + 1;
                k = fetch_coef<BN>(a, cc);
            }
            po.v[j] = pre_value<BN>(xin.v[j], k, no.v[j]);
            yo.v[j] = act_apply<ACT>(po.v[j]);
            ++rr;
        }
    }
    if constexpr (RES) {
#pragma unroll
        for (int j = 0; j < 4; ++j) yo.v[j] = with_residual(yo.v[j], rin.v[j], a.res_alpha, a.res_beta);
    }
    if (full) {
        if (a.x_saved) st<4, NT>(a.x_saved, e, xin);
        if (BN && a.x_norm) st<4, NT>(a.x_norm, e, no);
        if (a.pre) st<4, NT>(a.pre, e, po);
        st<4, NT>(a.y, e, yo);
    } else {
        for (int j = 0; j < 4 && e + j < a.total; ++j) {
            if (a.x_saved) a.x_saved[e + j] = xin.v[j];
            if (BN && a.x_norm) a.x_norm[e + j] = no.v[j];
            if (a.pre) a.pre[e + j] = po.v[j];
            a.y[e + j] = yo.v[j];
        }
    }
}

template<int ACT, bool BN, bool NT>
__global__ __launch_bounds__(kBlock) void epilogue_fwd_kernel(EpilogueArgs a)
{
    epilogue_fwd_body<ACT, BN, NT, false>(a);
}

// The same pass with the shortcut that follows the layer: one more stream read, no tensor in between.
template<int ACT, bool BN, bool NT>
__global__ __launch_bounds__(kBlock) void epilogue_shortcut_fwd_kernel(EpilogueArgs a)
{
    epilogue_fwd_body<ACT, BN, NT, true>(a);
}

// Pointers that are not 16-byte aligned: one element per lane.
template<int ACT, bool BN>
__global__ __launch_bounds__(kBlock) void epilogue_fwd_scalar_kernel(EpilogueArgs a)
{
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= a.total) return;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    const FoldCoef k = fetch_coef<BN>(a, c);
    const float x = a.x[e];
    float xn;
    const float pre = pre_value<BN>(x, k, xn);
    if (a.x_saved) a.x_saved[e] = x;
    if (BN && a.x_norm) a.x_norm[e] = xn;
    if (a.pre) a.pre[e] = pre;
    float y = act_apply<ACT>(pre);
    if (a.residual) y = with_residual(y, a.residual[e], a.res_alpha, a.res_beta);
    a.y[e] = y;
}

// ---- the inference epilogue with the 2 x 2, stride 2 max-pool that follows the layer ----
// A lane takes VX consecutive outputs of one output row: 2 * VX inputs of each of two input rows (one
// plane, so one channel's constants), applies the epilogue to them and keeps the largest of each window,
// compared in the order the pool's own kernel compares them.  The layer's own output is written only when
// something else reads it.
struct EpiloguePoolArgs {
    const float* x;
    float* y;             // nullable: the layer's own output
    float* pooled;
    const FoldCoef* table;
    uint32_t units;       // lanes with work
    uint32_t iw, ow;
    FastDiv by_owv;       // ow / VX
    FastDiv by_oh;
    FastDiv by_channels;
};

template<int ACT, int VX, bool NT>
__global__ __launch_bounds__(kBlock) void epilogue_pool2_fwd_kernel(EpiloguePoolArgs a)
{
    const uint32_t t = blockIdx.x * static_cast<uint32_t>(kBlock) + threadIdx.x;
    if (t >= a.units) return;
    uint32_t rows, oxv, plane, oy, q, c;
    a.by_owv.divmod(t, rows, oxv);
    a.by_oh.divmod(rows, plane, oy);
    a.by_channels.divmod(plane, q, c);
    const uint32_t ih = a.by_oh.d * 2;
    const uint32_t in0 = (plane * ih + 2 * oy) * a.iw + 2 * oxv * VX;      // < 2^31 checked by the host
    const Pack<2 * VX> r0 = ld<2 * VX, NT>(a.x, in0);
    const Pack<2 * VX> r1 = ld<2 * VX, NT>(a.x, in0 + a.iw);
    const FoldCoef k = a.table[c];
    Pack<2 * VX> y0, y1;
    float pre[2 * VX], xn;
#pragma unroll
    for (int j = 0; j < 2 * VX; ++j) pre[j] = pre_value<true>(r0.v[j], k, xn);
    act_apply_n<ACT>(pre, y0.v);
#pragma unroll
    for (int j = 0; j < 2 * VX; ++j) pre[j] = pre_value<true>(r1.v[j], k, xn);
    act_apply_n<ACT>(pre, y1.v);
    if (a.y) {
        st<2 * VX, NT>(a.y, in0, y0);
        st<2 * VX, NT>(a.y, in0 + a.iw, y1);
    }
    Pack<VX> best;
#pragma unroll
    for (int j = 0; j < VX; ++j) {
        float b = y0.v[2 * j];
        if (y0.v[2 * j + 1] > b) b = y0.v[2 * j + 1];
        if (y1.v[2 * j] > b) b = y1.v[2 * j];
        if (y1.v[2 * j + 1] > b) b = y1.v[2 * j + 1];
        best.v[j] = b;
    }
    st<VX, NT>(a.pooled, (plane * a.by_oh.d + oy) * a.ow + oxv * VX, best);
}

int check_shape(const char* who, int batch, int channels, int spatial, uint32_t* total)
{
    if (batch <= 0 || channels <= 0 || spatial <= 0)
        return fail_invalid("%s: batch, channels and spatial must be positive (%d, %d, %d)", who, batch, channels,
                            spatial);
    const unsigned long long t = 1ull * batch * channels * spatial;
    if (t >= (1ull << 31)) {
        set_error("%s: %llu elements; tensors of 2^31 elements or more are not supported", who, t);
        return PXH_ERR_UNSUPPORTED;
    }
    *total = static_cast<uint32_t>(t);
    return PXH_OK;
}

template<bool BN>
int launch_epilogue_fwd(const char* who, EpilogueArgs a, int activation, hipStream_t stream)
{
    // the walk across a plane boundary handles any plane size, including single elements
    const bool vec = aligned16(a.x) && aligned16(a.y) && aligned16(a.pre) && aligned16(a.x_saved) &&
                     aligned16(a.x_norm) && aligned16(a.residual);
    // bytes this launch moves: x in, y out, plus each materialised extra output and the shortcut's source
    const size_t streams = 2 + (a.pre ? 1 : 0) + (a.x_saved ? 1 : 0) + (a.x_norm ? 1 : 0) + (a.residual ? 1 : 0);
    const bool nt = static_cast<size_t>(a.total) * 4 * streams >= kStreamingBytes;
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (vec) {
            const dim3 grid(grid_for(a.total, static_cast<size_t>(kBlock) * 4));
            if (a.residual) {
                if (nt) hipLaunchKernelGGL((epilogue_shortcut_fwd_kernel<ACT, BN, true>), grid, dim3(kBlock), 0, stream, a);
                else hipLaunchKernelGGL((epilogue_shortcut_fwd_kernel<ACT, BN, false>), grid, dim3(kBlock), 0, stream, a);
            } else if (nt) hipLaunchKernelGGL((epilogue_fwd_kernel<ACT, BN, true>), grid, dim3(kBlock), 0, stream, a);
            else hipLaunchKernelGGL((epilogue_fwd_kernel<ACT, BN, false>), grid, dim3(kBlock), 0, stream, a);
        } else {
            hipLaunchKernelGGL((epilogue_fwd_scalar_kernel<ACT, BN>), dim3(grid_for(a.total, kBlock)),
                               dim3(kBlock), 0, stream, a);
        }
    });
    if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
    return check_launch(who);
}

// ------------------------------------------------------------------------------------------
// Per-channel reductions.
//
// Channel c owns `batch` planes of `spatial` contiguous floats.  A plane is cut into segments of
// kSeg floats; the (image, segment) items of a channel are dealt kItemsPerBlock to a workgroup,
// one item per wavefront at a time (64 lanes x 128-bit x 4 loads = one segment).  Lanes sum a
// segment in fp32, carry across segments in double; the workgroup's pair of sums goes to
// partial[c][j] and a second kernel adds the partials of a channel in a fixed order.
// ------------------------------------------------------------------------------------------
constexpr int kSegLoads = 4;                  // 128-bit loads in flight per lane
constexpr int kSeg = kWave * 4 * kSegLoads;   // 1024 floats
constexpr int kItemsPerBlock = 16;

struct ReduceGeom {
    int channels, spatial, parts, items, blocks;
    FastDiv by_parts;
    FastDiv by_blocks;
};

ReduceGeom make_geom(int batch, int channels, int spatial)
{
    ReduceGeom g;
    g.channels = channels;
    g.spatial = spatial;
    g.parts = (spatial + kSeg - 1) / kSeg;
    g.items = batch * g.parts;
    g.blocks = (g.items + kItemsPerBlock - 1) / kItemsPerBlock;
    g.by_parts = FastDiv(static_cast<uint32_t>(g.parts));
    g.by_blocks = FastDiv(static_cast<uint32_t>(g.blocks));
    return g;
}

// Calls body(base, seg0, seg1, lane) for every item of workgroup (c, j): `base` is the offset of
// the item's plane, [seg0, seg1) its segment inside the plane.
template<typename Body>
__device__ __forceinline__ void for_each_item(const ReduceGeom& g, uint32_t c, uint32_t j, Body&& body)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int first = j * kItemsPerBlock;
    const int last = min(first + kItemsPerBlock, g.items);
    for (int it = first + wave; it < last; it += kBlock / kWave) {
        uint32_t n, part;
        g.by_parts.divmod(static_cast<uint32_t>(it), n, part);
        const size_t base = (static_cast<size_t>(n) * g.channels + c) * g.spatial;
        const int seg0 = part * kSeg;
        const int seg1 = min(g.spatial, seg0 + kSeg);
        body(base, seg0, seg1, lane);
    }
}

// ---- statistics: S1 = sum(x - K), S2 = sum((x - K)^2), K = first element of the channel ----
template<int V, bool NT>
__global__ __launch_bounds__(kBlock) void bn_stats_partial_kernel(const float* x, ReduceGeom g, double2* partial)
{
    __shared__ double slots[2][kBlock / kWave];
    uint32_t c, j;
    g.by_blocks.divmod(blockIdx.x, c, j);
    const float shift = x[static_cast<size_t>(c) * g.spatial];
    double s1 = 0.0, s2 = 0.0;
    for_each_item(g, c, j, [&](size_t base, int seg0, int seg1, int lane) {
        constexpr int kLoads = kSeg / (kWave * V);
        Pack<V> v[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) v[u] = ld<V, NT>(x, base + off);
        }
        float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) {
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    const float d = v[u].v[k] - shift;
                    a1 += d;
                    a2 += d * d;
                }
            }
        }
        s1 += static_cast<double>(a1);
        s2 += static_cast<double>(a2);
    });
    const double t1 = block_sum(s1, slots[0]);
    const double t2 = block_sum(s2, slots[1]);
    if (threadIdx.x == 0) partial[blockIdx.x] = make_double2(t1, t2);
}

// Mean / variance from the shifted sums S1 = sum(x - K), S2 = sum((x - K)^2) over `count` values,
// and the rolling statistics moved towards them.
struct ChannelStats { float mean, var, rolling_mean, rolling_var; };

__device__ __forceinline__ ChannelStats channel_stats(double s1, double s2, float shift_value, double count,
                                                      float rolling_mean, float rolling_var)
{
    const double shift = static_cast<double>(shift_value);
    const double m = s1 / count;
    double v = (s2 - s1 * m) / count;
    if (v < 0.0) v = 0.0;
    ChannelStats st;
    st.mean = static_cast<float>(shift + m);
    st.var = static_cast<float>(v);
    // sscal then saxpy: two fp32 roundings each (src/BatchNorm.cpp:53-56)
    float r = 0.99f * rolling_mean;
    st.rolling_mean = r + .01f * st.mean;
    r = 0.99f * rolling_var;
    st.rolling_var = r + .01f * st.var;
    return st;
}

// The same for channel c of the tensors: writes the statistics and folds the constants the apply
// pass needs.
__device__ __forceinline__ FoldCoef finish_stats(double s1, double s2, float shift_value, double count, int c,
                                                 float* mean, float* var, float* rolling_mean, float* rolling_var,
                                                 const float* scale, const float* bias)
{
    const ChannelStats st = channel_stats(s1, s2, shift_value, count, rolling_mean ? rolling_mean[c] : 0.0f,
                                          rolling_var ? rolling_var[c] : 0.0f);
    mean[c] = st.mean;
    var[c] = st.var;
    if (rolling_mean) {
        rolling_mean[c] = st.rolling_mean;
        rolling_var[c] = st.rolling_var;
    }
    return make_coef(st.mean, st.var, scale ? scale[c] : 1.0f, bias ? bias[c] : 0.0f);
}

// One wavefront per channel adds the channel's partials and finishes the statistics.
__global__ __launch_bounds__(kBlock) void bn_stats_finish_kernel(const float* x, const double2* partial, int channels,
                                                                 int spatial, int blocks, double count, float* mean,
                                                                 float* var, float* rolling_mean, float* rolling_var,
                                                                 const float* scale, const float* bias,
                                                                 FoldCoef* table)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int c = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (c >= channels) return;
    double s1 = 0.0, s2 = 0.0;
    for (int j = lane; j < blocks; j += kWave) {
        const double2 p = partial[static_cast<size_t>(c) * blocks + j];
        s1 += p.x;
        s2 += p.y;
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if (lane == 0) {
        const FoldCoef k = finish_stats(s1, s2, x[static_cast<size_t>(c) * spatial], count, c, mean, var, rolling_mean,
                                        rolling_var, scale, bias);
        if (table) table[c] = k;
    }
}

// ---- Layer::backward's gradient rescale + clip in front of the backward sums ----
// The layer's backward opens with the norm of its delta, a rescale when the norm is beyond a threshold
// and a clamp (include/Layer.h:385-397, 479-499), and only then runs the activation gradient and the
// batch-norm backward (include/ConvLayer.h:238-252).  The first pass over the delta can carry the sum
// of squares and the largest magnitude along with its own sums, which saves the read that the norm
// alone would cost; the decision is formed on the device (ClipPlan) and the later kernels follow it.
struct __attribute__((aligned(16))) ClipPlan {
    float norm, factor, clip;
    int work;       // 0: no value of the delta changes; kChanges: some do; | kClamps: and the clamp may move one
};
enum { kChanges = 1, kClamps = 2 };

// The plan from `count` partial (sum of squares, largest magnitude) pairs, added in an order that
// depends on THREADS alone: every workgroup that forms it arrives at the same one.  All THREADS
// threads of the workgroup call it; every one returns the plan.
template<int THREADS>
__device__ __forceinline__ ClipPlan clip_plan_from(const double2* part, int count, float threshold, float clip)
{
    __shared__ double plan_sums[THREADS / kWave];
    __shared__ float plan_tops[THREADS / kWave];
    double s = 0.0;
    float top = 0.0f;
    // kPlanLoads partials per thread and round, their loads in flight together (one after the other each
    // costs a trip to memory: 45 of them per thread at 16 x 32 x 608^2 with 256 threads)
    constexpr int kPlanLoads = 8;
    if (count <= THREADS) {
        // the one-launch backward's per-channel figures: one load per thread, the same sum
        const bool valid = static_cast<int>(threadIdx.x) < count;
        const double2 p = part[valid ? threadIdx.x : 0];
        s = valid ? p.x : 0.0;
        top = valid ? static_cast<float>(p.y) : 0.0f;
    } else for (int base = 0; base < count; base += THREADS * kPlanLoads) {
        double2 p[kPlanLoads];
#pragma unroll
        for (int u = 0; u < kPlanLoads; ++u) {
            const int j = base + u * THREADS + static_cast<int>(threadIdx.x);
            p[u] = part[j < count ? j : 0];
        }
#pragma unroll
        for (int u = 0; u < kPlanLoads; ++u) {
            const bool valid = base + u * THREADS + static_cast<int>(threadIdx.x) < count;
            s += valid ? p[u].x : 0.0;
            top = fmaxf(top, valid ? static_cast<float>(p[u].y) : 0.0f);
        }
    }
    s = wave_sum(s);
    top = wave_max(top);
    __syncthreads();       // the arrays may still be read from an earlier call
    if ((threadIdx.x & (kWave - 1)) == 0) {
        plan_sums[threadIdx.x / kWave] = s;
        plan_tops[threadIdx.x / kWave] = top;
    }
    __syncthreads();
    double total = 0.0;
    float peak = 0.0f;
#pragma unroll
    for (int w = 0; w < THREADS / kWave; ++w) {
        total += plan_sums[w];
        peak = fmaxf(peak, plan_tops[w]);
    }
    const RescalePlan r = plan_from_totals(total, peak, threshold, clip);
    return ClipPlan{ r.norm, r.factor, clip, (r.work ? kChanges : 0) | (r.clamps ? kClamps : 0) };
}

// What the clipped forms add to a launch: where the first pass leaves its norm partials, and the
// plan that the finish kernel of the first pass writes and everything after it reads.
struct ClipArgs {
    double2* norm_partial;     // [workgroups of the first pass]
    ClipPlan* plan;
    float threshold, clip;
    float* norm_out;           // nullable
};

constexpr int kPlanThreads = 1024;
constexpr int kRedoWorkgroups = 256;      // of the one-launch form's second launch

// The passes of a backward:  kPlain -- no rescale + clip in front;  kFirst -- the sums as if nothing
// had to change, plus the norm partials;  kRedo -- after the plan: leaves at once when the sums of the
// first pass still serve, else forms them again from the rescaled and clamped delta.
// The sums of the first pass serve when nothing changes, and for the batch-norm backward also when the
// delta is only rescaled (the clamp moves no value): they are linear in the delta, so the finish
// kernel multiplies them by the factor and the dx pass applies the factor to the delta it reads.
enum { kPlain = 0, kFirst = 1, kRedo = 2 };

// ---- backward sums: A = sum d', B = sum d' * (x - mean), d' = delta * act'(pre) ----
struct BackwardArgs {
    float* delta;
    const float* x;          // saved conv output (BN) or nullptr (bias only)
    const float* pre;        // nullable when BN: recomputed from x
    const float* mean;
    const float* var;
    const float* scale;
    const float* bias;
};

// WRITE (the bias-only layer, which has no dx pass): d' goes back into delta.  With kFirst nothing is
// written (the delta is still needed as it came); with kRedo the pass also runs, writing, when nothing
// has to change but the activation has a gradient to apply.
template<int ACT, bool BN, bool WRITE, int V, bool NT, int MODE = kPlain>
__global__ __launch_bounds__(kBlock) void bwd_partial_kernel(BackwardArgs a, ReduceGeom g, double2* partial,
                                                             ClipArgs clip = ClipArgs{})
{
    static_assert(!(WRITE && MODE == kFirst), "the first pass of a clipped backward leaves the delta alone");
    __shared__ double slots[2][kBlock / kWave];
    [[maybe_unused]] float factor = 1.0f, limit = 0.0f;
    [[maybe_unused]] bool changes = false;
    if constexpr (MODE == kRedo) {
        const ClipPlan plan = *clip.plan;
        changes = plan.work != 0;
        // the writing form has the delta to rewrite whenever a value changes; the other only its sums to
        // form again, and only when the clamp takes part
        const bool again = WRITE ? changes : (plan.work & kClamps) != 0;
        if (!again && !(WRITE && ACT != PXH_LINEAR)) return;
        factor = changes ? plan.factor : 1.0f;
        limit = changes ? plan.clip : 0.0f;
    }
    uint32_t c, j;
    g.by_blocks.divmod(blockIdx.x, c, j);
    FoldCoef k;
    if constexpr (BN) k = make_coef(a.mean[c], a.var[c], a.scale[c], a.bias[c]);
    const bool recompute = BN && a.pre == nullptr;
    double sa = 0.0, sb = 0.0;
    [[maybe_unused]] double sq = 0.0;
    [[maybe_unused]] float peak = 0.0f;
    for_each_item(g, c, j, [&](size_t base, int seg0, int seg1, int lane) {
        constexpr int kLoads = kSeg / (kWave * V);
        Pack<V> d[kLoads], xv[kLoads], pv[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) {
                d[u] = ld<V, NT>(a.delta, base + off);
                if constexpr (BN) xv[u] = ld<V, NT>(a.x, base + off);
                if constexpr (ACT != PXH_LINEAR) {
                    if (!recompute) pv[u] = ld<V, NT>(a.pre, base + off);
                }
            }
        }
        float fa = 0.0f, fb = 0.0f;
        [[maybe_unused]] float fq = 0.0f;
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) {
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    float dv = d[u].v[q];
                    if constexpr (MODE == kFirst) {
                        fq += dv * dv;
                        peak = fmaxf(peak, fabsf(dv));
                    }
                    if constexpr (MODE == kRedo) {
                        dv = rescaled_clipped(dv, factor, limit);
                        d[u].v[q] = dv;
                    }
                    if constexpr (ACT != PXH_LINEAR) {
                        float pre;
                        if (recompute) pre = affine(normalize(xv[u].v[q], k), k);
                        else pre = pv[u].v[q];
                        dv = dv * act_grad<ACT>(pre);
                        d[u].v[q] = dv;
                    }
                    fa += dv;
                    if constexpr (BN) fb += dv * (xv[u].v[q] - k.mean);
                }
                if constexpr (WRITE && (ACT != PXH_LINEAR || MODE == kRedo)) {
                    if (ACT != PXH_LINEAR || changes) st<V, NT>(a.delta, base + off, d[u]);
                }
            }
        }
        sa += static_cast<double>(fa);
        sb += static_cast<double>(fb);
        if constexpr (MODE == kFirst) sq += static_cast<double>(fq);
    });
    const double ta = block_sum(sa, slots[0]);
    const double tb = block_sum(sb, slots[1]);
    if (threadIdx.x == 0) partial[blockIdx.x] = make_double2(ta, tb);
    if constexpr (MODE == kFirst) {
        __shared__ float peaks[kBlock / kWave];
        const double tq = block_sum(sq, slots[0]);      // synchronises before it reuses the slots
        peak = wave_max(peak);
        if ((threadIdx.x & (kWave - 1)) == 0) peaks[threadIdx.x / kWave] = peak;
        __syncthreads();
        if (threadIdx.x == 0) {
            float top = peaks[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) top = fmaxf(top, peaks[w]);
            clip.norm_partial[blockIdx.x] = make_double2(tq, static_cast<double>(top));
        }
    }
}

// Per-channel constants of the dx pass, produced by the finish kernel (64 bytes).
struct __attribute__((aligned(16))) DxCoef {
    FoldCoef f;
    double rroot;     // 1 / sqrt(float(var + eps))
    double c2;        // var_delta * 2 / count
    double md_term;   // float(mean_delta / float(count))
    double pad;
};

// What the sums A = sum d' and B = sum d' * (x - mean) of a channel amount to: the additions to its two
// parameter updates, its mean and variance deltas, and the constants of the dx pass.  Arithmetic only.
struct FinishedChannel {
    DxCoef k;
    float bias_add, scale_add, mean_delta, var_delta;
};

template<bool BN>
__device__ __forceinline__ FinishedChannel finished_channel(double sa, double sb, int count, const FoldCoef& f, float v,
                                                            float s)
{
    FinishedChannel r{};
    r.bias_add = static_cast<float>(sa);
    if constexpr (BN) {
        // sum d' * x_hat with x_hat = (x - mean) / (sqrt(var) + eps)
        const double denom = sqrt(static_cast<double>(v)) + static_cast<double>(kEps);
        r.scale_add = static_cast<float>(sb / denom);
        // sums of d'' = d' * scale
        const float sum_dd = static_cast<float>(sa * static_cast<double>(s));
        const float sum_ddx = static_cast<float>(sb * static_cast<double>(s));
        const float ve = v + kEps;
        r.mean_delta = static_cast<float>(static_cast<double>(sum_dd) * (-1. / static_cast<double>(sqrtf(ve))));
        r.var_delta = sum_ddx * (-.5f * powf(ve, -3.0f / 2.0f));
        r.k.f = f;
        r.k.rroot = 1.0 / sqrt(static_cast<double>(ve));
        r.k.c2 = static_cast<double>(r.var_delta) * 2. / static_cast<double>(count);
        r.k.md_term = static_cast<double>(r.mean_delta / static_cast<float>(count));
        r.k.pad = 0.0;
    }
    return r;
}

// Channel c from its sums: accumulates the parameter updates and returns the constants of the dx pass.
template<bool BN>
__device__ __forceinline__ DxCoef finish_backward(double sa, double sb, int c, int count, const float* mean,
                                                  const float* var, const float* scale, const float* bias,
                                                  float* scale_updates, float* bias_updates, float* mean_delta,
                                                  float* var_delta)
{
    // every load before the first store: a load behind a store waits for that store as well
    FoldCoef f{};
    float v = 0.0f, s = 0.0f, scale_updates_in = 0.0f;
    const float bias_updates_in = bias_updates[c];
    if constexpr (BN) {
        scale_updates_in = scale_updates[c];
        v = var[c];
        s = scale[c];
        f = make_coef(mean[c], v, s, bias[c]);
    }
    const FinishedChannel r = finished_channel<BN>(sa, sb, count, f, v, s);
    bias_updates[c] = bias_updates_in + r.bias_add;
    if constexpr (BN) {
        scale_updates[c] = scale_updates_in + r.scale_add;
        if (mean_delta) mean_delta[c] = r.mean_delta;
        if (var_delta) var_delta[c] = r.var_delta;
    }
    return r.k;
}

// kFirst (workgroups of kPlanThreads): every workgroup forms the plan from all norm partials of the first
// pass (the same additions in the same order everywhere), the first one records it, and the channels
// are finished only when nothing has to change; kRedo: finishes them from the second pass's sums when
// something had to.
template<bool BN, int MODE = kPlain, int THREADS = kBlock>
__global__ __launch_bounds__(THREADS) void bwd_finish_kernel(const double2* partial, int channels, int blocks, int count,
                                                             const float* mean, const float* var, const float* scale,
                                                             const float* bias, float* scale_updates,
                                                             float* bias_updates, float* mean_delta, float* var_delta,
                                                             DxCoef* coef, ClipArgs clip = ClipArgs{})
{
    [[maybe_unused]] double sums_factor = 1.0;
    if constexpr (MODE == kFirst) {
        const ClipPlan plan = clip_plan_from<THREADS>(clip.norm_partial, channels * blocks, clip.threshold, clip.clip);
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            *clip.plan = plan;
            if (clip.norm_out) *clip.norm_out = plan.norm;
        }
        // with batch-norm the sums serve unless the clamp takes part; a bias-only layer's delta is
        // rewritten by the second pass whenever a value changes, and that pass leaves exact sums
        if (BN ? (plan.work & kClamps) != 0 : plan.work != 0) return;
        sums_factor = static_cast<double>(plan.factor);
    }
    if constexpr (MODE == kRedo) {
        const int work = clip.plan->work;
        if (BN ? (work & kClamps) == 0 : work == 0) return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const int c = blockIdx.x * (THREADS / kWave) + threadIdx.x / kWave;
    if (c >= channels) return;
    double sa = 0.0, sb = 0.0;
    for (int j = lane; j < blocks; j += kWave) {
        const double2 p = partial[static_cast<size_t>(c) * blocks + j];
        sa += p.x;
        sb += p.y;
    }
    sa = wave_sum(sa);
    sb = wave_sum(sb);
    if constexpr (MODE == kFirst) {
        if (sums_factor != 1.0) {
            sa *= sums_factor;
            sb *= sums_factor;
        }
    }
    if (lane == 0) {
        const DxCoef k = finish_backward<BN>(sa, sb, c, count, mean, var, scale, bias, scale_updates, bias_updates,
                                             mean_delta, var_delta);
        if constexpr (BN) coef[c] = k;
    }
}

struct DxArgs {
    float* delta;
    const float* x;
    const float* pre;   // nullable: recomputed
    const DxCoef* coef;
    FastDiv by_spatial;
    FastDiv by_channels;
    uint32_t total;
    const ClipPlan* plan;     // the clipped form: the delta goes through the plan's rescale + clamp first
};

// The delta as the sums saw it: through the plan when there is one and it changes anything.
template<bool CLIPPED, int V>
__device__ __forceinline__ void apply_plan(const DxArgs& a, Pack<V>& d)
{
    if constexpr (CLIPPED) {
        const ClipPlan plan = *a.plan;
        if (plan.work) {
#pragma unroll
            for (int k = 0; k < V; ++k) d.v[k] = rescaled_clipped(d.v[k], plan.factor, plan.clip);
        }
    }
}

template<int ACT>
__device__ __forceinline__ float dx_value(float d, float x, float pre_in, bool recompute, const DxCoef& k)
{
    if constexpr (ACT != PXH_LINEAR) {
        float pre = pre_in;
        if (recompute) pre = affine(normalize(x, k.f), k.f);
        d = d * act_grad<ACT>(pre);
    }
    const float dd = d * k.f.scale;
    const float xm = x - k.f.mean;
    // src/CpuUtil.cpp:336-338 evaluated in double, stored as float
    const double v = static_cast<double>(dd) * k.rroot + k.c2 * static_cast<double>(xm) + k.md_term;
    return static_cast<float>(v);
}

template<int ACT, bool NT, bool CLIPPED = false>
__global__ __launch_bounds__(kBlock) void bn_dx_kernel(DxArgs a)
{
    const uint32_t e = (blockIdx.x * static_cast<uint32_t>(kBlock) + threadIdx.x) * 4;
    if (e >= a.total) return;
    const bool full = e + 3 < a.total;
    const bool recompute = a.pre == nullptr;
    Pack<4> din, xin, pin;
    if (full) {
        din = ld<4, NT>(a.delta, e);
        xin = ld<4, NT>(a.x, e);
        if (ACT != PXH_LINEAR && !recompute) pin = ld<4, NT>(a.pre, e);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const bool ok = e + k < a.total;
            din.v[k] = ok ? a.delta[e + k] : 0.0f;
            xin.v[k] = ok ? a.x[e + k] : 0.0f;
            pin.v[k] = (ok && ACT != PXH_LINEAR && !recompute) ? a.pre[e + k] : 0.0f;
        }
    }
    apply_plan<CLIPPED, 4>(a, din);
    const uint32_t hw = a.by_spatial.d;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    Pack<4> out;
    const bool crosses = !(r + 3 < hw);
    if (!__ballot(crosses)) {
        const DxCoef k = a.coef[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) out.v[j] = dx_value<ACT>(din.v[j], xin.v[j], pin.v[j], recompute, k);
    } else if (hw >= 4) {
        // one boundary per vector at most: constants selected per element, one copy of the arithmetic
        // for the wave (see epilogue_fwd_kernel)
        const DxCoef k0 = a.coef[c];
        DxCoef k1 = k0;
        if (crosses) k1 = a.coef[c + 1 == a.by_channels.d ? 0 : c + 1];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool here = r + j < hw;
            DxCoef k;
            k.f.mean = here ? k0.f.mean : k1.f.mean;
            k.f.r_hi = here ? k0.f.r_hi : k1.f.r_hi;
            k.f.r_lo = here ? k0.f.r_lo : k1.f.r_lo;
            k.f.scale = here ? k0.f.scale : k1.f.scale;
            k.f.bias = here ? k0.f.bias : k1.f.bias;
            k.rroot = here ? k0.rroot : k1.rroot;
            k.c2 = here ? k0.c2 : k1.c2;
            k.md_term = here ? k0.md_term : k1.md_term;
            out.v[j] = dx_value<ACT>(din.v[j], xin.v[j], pin.v[j], recompute, k);
        }
    } else {
        uint32_t rr = r, cc = c;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (rr == hw) {
                rr = 0;
                cc = cc + 1 == a.by_channels.d ? 0 : cc + 1;
            }
            out.v[j] = dx_value<ACT>(din.v[j], xin.v[j], pin.v[j], recompute, a.coef[cc]);
            ++rr;
        }
    }
    if (full) {
        st<4, NT>(a.delta, e, out);
    } else {
        for (int j = 0; j < 4 && e + j < a.total; ++j) a.delta[e + j] = out.v[j];
    }
}

template<int ACT, bool CLIPPED = false>
__global__ __launch_bounds__(kBlock) void bn_dx_scalar_kernel(DxArgs a)
{
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= a.total) return;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    const bool recompute = a.pre == nullptr;
    const float pre = (ACT != PXH_LINEAR && !recompute) ? a.pre[e] : 0.0f;
    Pack<1> d;
    d.v[0] = a.delta[e];
    apply_plan<CLIPPED, 1>(a, d);
    a.delta[e] = dx_value<ACT>(d.v[0], a.x[e], pre, recompute, a.coef[c]);
}

// ---------------------------------------------------------------- channel-resident training passes
// For a tensor whose per-channel slice (batch * spatial floats) fits the registers of one
// workgroup, the three launches above (partial sums, finish, apply) collapse into one: workgroup c
// holds channel c, reduces it, finishes the statistics and applies them.  The tensor is read from
// memory once, and a small layer costs one launch instead of three.
constexpr int kResidentThreads = 1024;
// The scalar forms also come with workgroups of half the size, four to a compute unit instead of two:
// for the layers with a thousand channels of 19 x 19, whose workgroups would otherwise run in two rounds.
constexpr int kResidentNarrowThreads = 512;

// Sum of two doubles over the workgroup; every thread returns both totals.
template<int T>
__device__ __forceinline__ void resident_sum2(double& a, double& b, double (*slots)[T / kWave])
{
    a = wave_sum(a);
    b = wave_sum(b);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) {
        slots[0][wave] = a;
        slots[1][wave] = b;
    }
    __syncthreads();
    double ta = 0.0, tb = 0.0;
#pragma unroll
    for (int w = 0; w < T / kWave; ++w) {
        ta += slots[0][w];
        tb += slots[1][w];
    }
    a = ta;
    b = tb;
}

// The same for a workgroup of half the size whose thread t stands in for threads t and t + T of a workgroup
// of 2 T threads (sums a of the first, b of the second): the additions of resident_sum2<2 * T>, in its order.
template<int T>
__device__ __forceinline__ void resident_sum2_twin(double& a1, double& a2, double b1, double b2,
                                                   double (*slots)[2 * T / kWave])
{
    a1 = wave_sum(a1);
    a2 = wave_sum(a2);
    b1 = wave_sum(b1);
    b2 = wave_sum(b2);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) {
        slots[0][wave] = a1;
        slots[1][wave] = a2;
        slots[0][wave + T / kWave] = b1;
        slots[1][wave + T / kWave] = b2;
    }
    __syncthreads();
    double ta = 0.0, tb = 0.0;
#pragma unroll
    for (int w = 0; w < 2 * T / kWave; ++w) {
        ta += slots[0][w];
        tb += slots[1][w];
    }
    a1 = ta;
    a2 = tb;
}

// The same for three sums and a maximum (the first pass of a clipped backward).
template<int T>
__device__ __forceinline__ void resident_sum3_max(double& a, double& b, double& q, float& top,
                                                  double (*slots)[T / kWave], float* tops)
{
    a = wave_sum(a);
    b = wave_sum(b);
    q = wave_sum(q);
    top = wave_max(top);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) {
        slots[0][wave] = a;
        slots[1][wave] = b;
        slots[2][wave] = q;
        tops[wave] = top;
    }
    __syncthreads();
    double ta = 0.0, tb = 0.0, tq = 0.0;
    float tt = 0.0f;
    // four waves' figures at a time: all sixteen at once are 100 registers of LDS loads in flight
#pragma unroll 4
    for (int w = 0; w < T / kWave; ++w) {
        ta += slots[0][w];
        tb += slots[1][w];
        tq += slots[2][w];
        tt = fmaxf(tt, tops[w]);
    }
    a = ta;
    b = tb;
    q = tq;
    top = tt;
}

struct ResidentGeom {
    int channels, spatial;
    uint32_t per_channel;     // batch * spatial
    FastDiv by_spatial;
    // offset of element e of channel c's slice (e counts through the images)
    __device__ __forceinline__ size_t at(uint32_t c, uint32_t e) const
    {
        uint32_t n, r;
        by_spatial.divmod(e, n, r);
        return (static_cast<size_t>(n) * channels + c) * spatial + r;
    }
};

struct ResidentFwdArgs {
    const float* x;
    float* y;
    float* pre;        // nullable
    float* x_saved;    // nullable
    float* x_norm;     // nullable
    float* mean;
    float* var;
    float* rolling_mean;
    float* rolling_var;
    const float* scale;
    const float* bias;
    ResidentGeom g;
    // the shortcut that follows the layer (else null), as in EpilogueArgs
    const float* residual;
    float res_alpha, res_beta;
};

// A thread keeps R vectors in registers and L more in LDS (dynamic, L * kResidentThreads vectors:
// thread-major, so every access is the conflict-free 128-bit one).
template<int V, int R>
__device__ __forceinline__ Pack<V>* resident_lds_slot(float* lds, int r)
{
    return reinterpret_cast<Pack<V>*>(lds) + static_cast<size_t>(r - R) * kResidentThreads + threadIdx.x;
}

// Steps of the shortcut's source that a lane of the large form asks for before the reduction.  (The form with
// eight 128-bit vectors in registers and two workgroups per compute unit has no register to spare for any:
// 16 x 512 x 38^2 takes 32.9 us with four steps ahead against 31.0 us with none.)
constexpr int kResidualAhead = 4;

// V = 4 needs spatial % 4 == 0 and 16-byte aligned tensors.  R + L vectors per thread at most.
template<int ACT, int V, int R, int L, int T = kResidentThreads, bool RES = false>
__global__ __launch_bounds__(T, L == 0 && V * R <= 32 ? 8 : 4) void bn_resident_fwd_kernel(ResidentFwdArgs a)
{
    static_assert(L == 0 || T == kResidentThreads, "the LDS part is laid out for the full workgroup");
    extern __shared__ __align__(16) float resident_lds[];
    // The 128-bit form with workgroups of half the size adds a channel up exactly as the full workgroups do,
    // so that a layer gives the same statistics to the bit with and without a shortcut riding on it: thread t
    // keeps the sums of the full form's threads t (even steps) and t + T (odd steps) apart.
    constexpr bool kTwin = V == 4 && T < kResidentThreads;
    static_assert(!kTwin || 2 * T == kResidentThreads, "half the size");
    __shared__ double slots[2][(kTwin ? 2 : 1) * T / kWave];
    __shared__ FoldCoef shared_coef;
    const uint32_t c = blockIdx.x;
    const float shift = a.x[static_cast<size_t>(c) * a.g.spatial];
    // issued now, needed after the reduction
    const float rm_in = a.rolling_mean[c], rv_in = a.rolling_var[c], scale_in = a.scale[c], bias_in = a.bias[c];
    Pack<V> v[R];
    float a1 = 0.0f, a2 = 0.0f;
    [[maybe_unused]] float b1 = 0.0f, b2 = 0.0f;
    // Every tensor here is touched once and goes past the caches (non-temporal: with the whole slice
    // of every channel asked for at once, cached reads run at two thirds of the rate; the backward
    // kernel keeps x cached, which it reads twice).
    // No branch around a load: a lane past the end of the slice reads the slice's first vector and
    // adds nothing, so that the loads of a lane are in flight together (behind a branch each one is
    // waited for before the next is issued, and a wave then has one kilobyte on its way at a time).
    const auto element = [&](int r) { return static_cast<uint32_t>(r * T + threadIdx.x) * V; };
    const auto fetch = [&](int r) {
        const uint32_t e = element(r);
        return ld<V, true>(a.x, a.g.at(c, e < a.g.per_channel ? e : 0u));
    };
    const auto add = [&](int r, const Pack<V>& t) {
        const bool valid = element(r) < a.g.per_channel;
        const bool second = kTwin && (r & 1);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const float d = t.v[k] - shift;
            if (second) {
                b1 += valid ? d : 0.0f;
                b2 += valid ? d * d : 0.0f;
            } else {
                a1 += valid ? d : 0.0f;
                a2 += valid ? d * d : 0.0f;
            }
        }
    };
    // the LDS part first, all of it at once: its registers are free again before the register part
    // is loaded, which lands where it stays
    if constexpr (L > 0) {
        Pack<V> stage[L];
#pragma unroll
        for (int r = R + L - 1; r >= R; --r) stage[r - R] = fetch(r);
#pragma unroll
        for (int r = R + L - 1; r >= R; --r) {
            add(r, stage[r - R]);
            *resident_lds_slot<V, R>(resident_lds, r) = stage[r - R];
        }
        // the sums as they stand, before the registers are handed to the second part
        asm volatile("" : "+v"(a1), "+v"(a2));
    }
#pragma unroll
    for (int r = R - 1; r >= 0; --r) v[r] = fetch(r);
    // The shortcut's source does not wait for the statistics: its first steps are asked for now, behind the
    // slice's own loads, and arrive while the sums are formed -- all of them where a lane holds few values
    // (16 x 1024 x 19^2: 19.9 us against 25.6 us with every step's load behind the reduction).
    // (the half-size workgroups of the 128-bit form have 128 registers: eight of twelve steps, four of sixteen)
    constexpr int kAhead = !RES ? 0 : V * (R + L) <= 8 ? R + L : L > 0 ? kResidualAhead
                                : T < kResidentThreads ? (R <= 12 ? 8 : 4) : 0;
    [[maybe_unused]] Pack<V> ahead[kAhead > 0 ? kAhead : 1];
    if constexpr (RES) {
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const uint32_t e = element(i);
            ahead[i] = ld<V, true>(a.residual, a.g.at(c, e < a.g.per_channel ? e : 0u));
        }
    }
#pragma unroll
    for (int r = R - 1; r >= 0; --r) add(r, v[r]);
    double s1 = static_cast<double>(a1), s2 = static_cast<double>(a2);
    if constexpr (kTwin) resident_sum2_twin<T>(s1, s2, static_cast<double>(b1), static_cast<double>(b2), slots);
    else resident_sum2<T>(s1, s2, slots);
    if (threadIdx.x == 0) {
        const ChannelStats st = channel_stats(s1, s2, shift, static_cast<double>(a.g.per_channel), rm_in, rv_in);
        a.mean[c] = st.mean;
        a.var[c] = st.var;
        a.rolling_mean[c] = st.rolling_mean;
        a.rolling_var[c] = st.rolling_var;
        shared_coef = make_coef(st.mean, st.var, scale_in, bias_in);
    }
    __syncthreads();
    const FoldCoef k = shared_coef;
    const auto apply = [&](int r, [[maybe_unused]] const Pack<V>& from) {
        const uint32_t e = (r * T + threadIdx.x) * V;
        if (e < a.g.per_channel) {
            const size_t where = a.g.at(c, e);
            const Pack<V> t = r < R ? v[r < R ? r : 0] : *resident_lds_slot<V, R>(resident_lds, r);
            Pack<V> xn, pre, out;
#pragma unroll
            for (int q = 0; q < V; ++q) {
                xn.v[q] = normalize(t.v[q], k);
                pre.v[q] = affine(xn.v[q], k);
                out.v[q] = act_apply<ACT>(pre.v[q]);
                if constexpr (RES) out.v[q] = with_residual(out.v[q], from.v[q], a.res_alpha, a.res_beta);
            }
            if (a.x_saved) st<V, true>(a.x_saved, where, t);
            if (a.x_norm) st<V, true>(a.x_norm, where, xn);
            if (a.pre) st<V, true>(a.pre, where, pre);
            st<V, true>(a.y, where, out);
        }
    };
    if constexpr (RES) {
        // the rest of the shortcut's source four steps at a time, no branch around its loads (see above)
        constexpr int kGroup = 4;
        static_assert((R + L) % kGroup == 0 && kAhead % kGroup == 0, "steps come in whole groups");
#pragma unroll
        for (int first = 0; first < R + L; first += kGroup) {
            Pack<V> from[kGroup];
#pragma unroll
            for (int i = 0; i < kGroup; ++i) {
                if (first + i < kAhead) {
                    from[i] = ahead[first + i < kAhead ? first + i : 0];
                } else {
                    const uint32_t e = element(first + i);
                    from[i] = ld<V, true>(a.residual, a.g.at(c, e < a.g.per_channel ? e : 0u));
                }
            }
#pragma unroll
            for (int i = 0; i < kGroup; ++i) apply(first + i, from[i]);
        }
    } else {
#pragma unroll
        for (int r = 0; r < R + L; ++r) apply(r, Pack<V>{});
    }
}

struct ResidentBwdArgs {
    BackwardArgs b;
    float* scale_updates;
    float* bias_updates;
    float* mean_delta;   // nullable
    float* var_delta;    // nullable
    ResidentGeom g;
    // the clipped form (else null): per channel the (sum of squares, largest magnitude) of its delta,
    // the two sums it was finished with, and whether it was finished at all
    double2* channel_norm;
    double2* channel_sums;
    int* channel_done;
    ClipArgs clip;
};

// A channel that was finished with the sums (sa, sb) of its unscaled delta, after the plan turned out
// to rescale by `factor` (and its clamp to move nothing in this channel): everything the backward left
// is linear in the delta, so the accumulated updates get the difference and the two per-channel deltas
// are formed again.  The dx values are scaled by the caller.
__device__ __forceinline__ void rescale_finished_channel(double sa, double sb, double factor, int c, const float* var,
                                                         const float* scale, float* scale_updates,
                                                         float* bias_updates, float* mean_delta, float* var_delta)
{
    bias_updates[c] += static_cast<float>((factor - 1.0) * sa);
    const float v = var[c];
    const float s = scale[c];
    const double denom = sqrt(static_cast<double>(v)) + static_cast<double>(kEps);
    scale_updates[c] += static_cast<float>((factor - 1.0) * sb / denom);
    const float sum_dd = static_cast<float>(factor * sa * static_cast<double>(s));
    const float sum_ddx = static_cast<float>(factor * sb * static_cast<double>(s));
    const float ve = v + kEps;
    if (mean_delta) mean_delta[c] = static_cast<float>(static_cast<double>(sum_dd) * (-1. / static_cast<double>(sqrtf(ve))));
    if (var_delta) var_delta[c] = sum_ddx * (-.5f * powf(ve, -3.0f / 2.0f));
}

// The workgroup keeps d' = delta * act'(pre) (registers + LDS); x is read again for the dx phase
// (it is still in the cache: one channel's slice is a few hundred KB).
//
// With Layer::backward's rescale + clip in front (kFirst, then a kRedo launch of the same shape): the
// first launch also adds up the channel's squares and finds its largest magnitude.  The norm that
// decides the rescale is the whole tensor's and is not known inside the launch; but the factor is at
// most 1, so a channel whose own largest magnitude is within the clamp cannot be clamped whatever the
// factor turns out to be, and all it leaves is linear in its delta: it is finished as if nothing had
// to change.  A channel above the clamp is left untouched.  The kRedo launch forms the plan from the
// per-channel figures and leaves at once in the usual case (nothing to change); else a finished
// channel is scaled by the factor, and an untouched one runs the whole pass on the rescaled and
// clamped delta.
// Channel c of a backward whose first launch finished it with the sums of its unscaled delta, scaled
// by the factor the plan arrived at.
template<int V, int R, int L, int T>
__device__ __forceinline__ void resident_rescale_channel(const ResidentBwdArgs& a, uint32_t c, float factor)
{
#pragma unroll 1
    for (int r = 0; r < R + L; ++r) {
        const uint32_t e = (r * T + threadIdx.x) * V;
        if (e < a.g.per_channel) {
            const size_t where = a.g.at(c, e);
            Pack<V> t = ld<V, true>(a.b.delta, where);
#pragma unroll
            for (int q = 0; q < V; ++q) t.v[q] = factor * t.v[q];
            st<V, true>(a.b.delta, where, t);
        }
    }
    if (threadIdx.x == 0) {
        const double2 sums = a.channel_sums[c];
        rescale_finished_channel(sums.x, sums.y, static_cast<double>(factor), c, a.b.var, a.b.scale, a.scale_updates,
                                 a.bias_updates, a.mean_delta, a.var_delta);
    }
}

// Channel c by the whole workgroup; `factor` and `limit` are the plan's (kRedo only).
template<int ACT, int V, int R, int L, int MODE, int T>
__device__ __forceinline__ void resident_bwd_channel(const ResidentBwdArgs& a, const uint32_t c,
                                                     [[maybe_unused]] const float factor,
                                                     [[maybe_unused]] const float limit)
{
    extern __shared__ __align__(16) float resident_lds[];
    __shared__ double slots[MODE == kFirst ? 3 : 2][T / kWave];
    __shared__ DxCoef shared_coef;
    const FoldCoef k = make_coef(a.b.mean[c], a.b.var[c], a.b.scale[c], a.b.bias[c]);
    // The whole workgroup waits for the one thread that finishes the channel, so that thread's loads all
    // come before its first store (a load issued behind a store waits for that store too: one counter,
    // in order); the forms that run the short launches ask for them before the first pass, the large
    // form, which has no register to spare, when the sums are there.
    constexpr bool kEarly = L == 0;
    [[maybe_unused]] float early[3] = {};
    if constexpr (kEarly) {
        early[0] = a.bias_updates[c];
        early[1] = a.scale_updates[c];
        early[2] = a.b.var[c];
    }
    const auto finish = [&](double sa, double sb) {
        const float bias_updates_in = kEarly ? early[0] : a.bias_updates[c];
        const float scale_updates_in = kEarly ? early[1] : a.scale_updates[c];
        const float var_in = kEarly ? early[2] : a.b.var[c];
        const FinishedChannel r = finished_channel<true>(sa, sb, static_cast<int>(a.g.per_channel), k, var_in, k.scale);
        a.bias_updates[c] = bias_updates_in + r.bias_add;
        a.scale_updates[c] = scale_updates_in + r.scale_add;
        if (a.mean_delta) a.mean_delta[c] = r.mean_delta;
        if (a.var_delta) a.var_delta[c] = r.var_delta;
        return r.k;
    };
    const bool recompute = a.b.pre == nullptr;
    Pack<V> d[R];
    float fa = 0.0f, fb = 0.0f;
    [[maybe_unused]] float fq = 0.0f, peak = 0.0f;
    // Two shapes of the first pass.  Grouped: no branch around the loads (see the forward kernel), lanes
    // past the end read the first vector; kGroup steps at a time, their loads go out together, then each
    // is used as it arrives.  The large form (part of the slice in LDS) is bound by its loads and takes
    // them so in groups of four; the scalar form in groups of eight (behind a branch a lane waits for
    // each step's loads before it asks for the next: six trips to memory one after the other at
    // 16 x 256 x 19^2, 10.4 us against 8.8).  The 128-bit form without an LDS part is held to 64
    // registers, where a group of two already spills (18.3 against 16.4 us at 16 x 256 x 38^2): it skips a step
    // past the end of the slice outright, as every form does in the second pass, which finds x in the cache.
    constexpr int kGroup = L > 0 ? 4 : 8;
    constexpr bool kGrouped = L > 0 || V == 1;
    static_assert(!kGrouped || (R % kGroup == 0 && L % kGroup == 0), "steps come in whole groups");
    // `lane` is the thread index; the second pass takes it through an empty asm statement, so that
    // its addresses are formed again there instead of being held in registers (48 of them) from the first
    [[maybe_unused]] uint32_t lane = threadIdx.x;
    [[maybe_unused]] const auto element = [&](int r) { return (static_cast<uint32_t>(r * T) + lane) * V; };
    [[maybe_unused]] const auto place = [&](int r) {
        const uint32_t e = element(r);
        return a.g.at(c, e < a.g.per_channel ? e : 0u);
    };
    // one value of the delta on its way to d': the norm's share of it first (kFirst), or the plan's
    // rescale + clamp (kRedo), then the activation's gradient
    const auto prepared = [&](float t, float pre, bool valid) {
        if constexpr (MODE == kFirst) {
            fq += valid ? t * t : 0.0f;
            peak = fmaxf(peak, valid ? fabsf(t) : 0.0f);
        }
        if constexpr (MODE == kRedo) t = rescaled_clipped(t, factor, limit);
        if constexpr (ACT != PXH_LINEAR) t = t * act_grad<ACT>(pre);
        return t;
    };
    if constexpr (kGrouped) {
        // delta * f'(pre) in dv, and the step's share of the sums
        const auto take = [&](int r, Pack<V>& dv, const Pack<V>& xv, const Pack<V>& pv) {
            const bool valid = element(r) < a.g.per_channel;
#pragma unroll
            for (int q = 0; q < V; ++q) {
                const float t = prepared(dv.v[q], ACT != PXH_LINEAR ? pv.v[q] : 0.0f, valid);
                dv.v[q] = t;
                fa += valid ? t : 0.0f;
                fb += valid ? t * (xv.v[q] - k.mean) : 0.0f;
            }
        };
#pragma unroll
        for (int top = R + L - 1; top >= 0; top -= kGroup) {
            Pack<V> dv[kGroup], xv[kGroup], pv[kGroup];
            size_t where[kGroup];
#pragma unroll
            for (int i = 0; i < kGroup; ++i) {
                where[i] = place(top - i);
                dv[i] = ld<V, true>(a.b.delta, where[i]);
                xv[i] = ld<V, false>(a.b.x, where[i]);
            }
            // the pre-activation: the saved one, or formed again from x (one decision per group)
            if constexpr (ACT != PXH_LINEAR) {
                if (!recompute) {
#pragma unroll
                    for (int i = 0; i < kGroup; ++i) pv[i] = ld<V, true>(a.b.pre, where[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < kGroup; ++i) {
#pragma unroll
                        for (int q = 0; q < V; ++q) pv[i].v[q] = affine(normalize(xv[i].v[q], k), k);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < kGroup; ++i) {
                const int r = top - i;
                take(r, dv[i], xv[i], pv[i]);
                if (r < R) d[r < R ? r : 0] = dv[i];
                else *resident_lds_slot<V, R>(resident_lds, r) = dv[i];
            }
            // The group ends here for the compiler too: the sums are taken as they stand (otherwise it
            // puts the additions off to the end of the pass and keeps every group's values until then),
            // and the next group's loads stay behind this one's arithmetic -- either would need more
            // registers than a lane has.
            if constexpr (MODE == kFirst) asm volatile("" : "+v"(fa), "+v"(fb), "+v"(fq), "+v"(peak));
            else asm volatile("" : "+v"(fa), "+v"(fb));
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int r = R + L - 1; r >= 0; --r) {
            const uint32_t e = (r * T + lane) * V;
            if (e < a.g.per_channel) {
                const size_t where = a.g.at(c, e);
                Pack<V> dv = ld<V, true>(a.b.delta, where);
                const Pack<V> xv = ld<V, false>(a.b.x, where);
                Pack<V> pv;
                if constexpr (ACT != PXH_LINEAR) {
                    if (!recompute) pv = ld<V, true>(a.b.pre, where);
                }
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    float pre = 0.0f;
                    if constexpr (ACT != PXH_LINEAR) {
                        if (recompute) pre = affine(normalize(xv.v[q], k), k);
                        else pre = pv.v[q];
                    }
                    const float t = prepared(dv.v[q], pre, true);
                    dv.v[q] = t;
                    fa += t;
                    fb += t * (xv.v[q] - k.mean);
                }
                if (r < R) d[r < R ? r : 0] = dv;
                else *resident_lds_slot<V, R>(resident_lds, r) = dv;
            }
        }
    }
    double sa = static_cast<double>(fa), sb = static_cast<double>(fb);
    if constexpr (MODE == kFirst) {
        __shared__ float tops[T / kWave];
        __shared__ int finished;
        double sq = static_cast<double>(fq);
        resident_sum3_max<T>(sa, sb, sq, peak, slots, tops);
        if (threadIdx.x == 0) {
            const float lim = a.clip.clip;
            const bool within = !(lim > 0.0f) || (peak <= lim && sq == sq);
            finished = within ? 1 : 0;
            if (within) shared_coef = finish(sa, sb);
            a.channel_norm[c] = make_double2(sq, static_cast<double>(peak));
            a.channel_sums[c] = make_double2(sa, sb);
            a.channel_done[c] = within ? 1 : 0;
        }
        __syncthreads();
        if (!finished) return;
    } else {
        resident_sum2<T>(sa, sb, slots);
        if (threadIdx.x == 0) shared_coef = finish(sa, sb);
        __syncthreads();
    }
    const DxCoef kd = shared_coef;
    if constexpr (L > 0) {
        asm volatile("" : "+v"(lane));
#pragma unroll
        for (int first = 0; first < R + L; first += kGroup) {
            Pack<V> xv[kGroup];
#pragma unroll
            for (int i = 0; i < kGroup; ++i) xv[i] = ld<V, false>(a.b.x, place(first + i));
#pragma unroll
            for (int i = 0; i < kGroup; ++i) {
                const int r = first + i;
                const Pack<V> dv = r < R ? d[r < R ? r : 0] : *resident_lds_slot<V, R>(resident_lds, r);
                Pack<V> out;
#pragma unroll
                for (int q = 0; q < V; ++q) out.v[q] = dx_value<PXH_LINEAR>(dv.v[q], xv[i].v[q], 0.0f, false, kd);
                if (element(r) < a.g.per_channel) st<V, true>(a.b.delta, place(r), out);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        asm volatile("" : "+v"(lane));      // addresses formed again, not kept from the first pass
#pragma unroll
        for (int r = 0; r < R + L; ++r) {
            const uint32_t e = (r * T + lane) * V;
            if (e < a.g.per_channel) {
                const size_t where = a.g.at(c, e);
                const Pack<V> xv = ld<V, false>(a.b.x, where);
                const Pack<V> dv = r < R ? d[r < R ? r : 0] : *resident_lds_slot<V, R>(resident_lds, r);
                Pack<V> out;
#pragma unroll
                for (int q = 0; q < V; ++q) out.v[q] = dx_value<PXH_LINEAR>(dv.v[q], xv.v[q], 0.0f, false, kd);
                st<V, true>(a.b.delta, where, out);
            }
        }
    }
}
// One workgroup per channel.  (The forms without an LDS part are held to 64 registers, two workgroups
// per compute unit: they run the 19 x 19 and 38 x 38 layers, whose launches are too short to fill the
// machine with one.)  The workgroups of the kRedo launch form the plan from the per-channel figures of
// the first launch and leave at once when nothing has to change; the forms without an LDS part run it
// as a capped grid that walks the channels otherwise.
template<int ACT, int V, int R, int L, int MODE = kPlain, int T = kResidentThreads>
__global__ __launch_bounds__(T, L == 0 && MODE != kRedo ? 8 : 4) void bn_resident_bwd_kernel(ResidentBwdArgs a)
{
    static_assert(L == 0 || T == kResidentThreads, "the LDS part is laid out for the full workgroup");
    if constexpr (MODE == kRedo) {
        const ClipPlan plan = clip_plan_from<T>(a.channel_norm, a.g.channels, a.clip.threshold,
                                                               a.clip.clip);
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            *a.clip.plan = plan;
            if (a.clip.norm_out) *a.clip.norm_out = plan.norm;
        }
        if (!plan.work) return;
        if constexpr (L > 0) {
            // (one workgroup per channel: walking several costs the large form 450 bytes of spills per lane)
            const uint32_t c = blockIdx.x;
            if (!a.channel_done[c]) resident_bwd_channel<ACT, V, R, L, kRedo, T>(a, c, plan.factor, plan.clip);
            else if (plan.factor != 1.0f) resident_rescale_channel<V, R, L, T>(a, c, plan.factor);
        } else {
            for (uint32_t c = blockIdx.x; c < static_cast<uint32_t>(a.g.channels); c += gridDim.x) {
                if (!a.channel_done[c]) resident_bwd_channel<ACT, V, R, L, kRedo, T>(a, c, plan.factor, plan.clip);
                else if (plan.factor != 1.0f) resident_rescale_channel<V, R, L, T>(a, c, plan.factor);
                __syncthreads();       // the next channel reuses the workgroup's LDS
            }
        }
    } else {
        resident_bwd_channel<ACT, V, R, L, MODE, T>(a, blockIdx.x, 1.0f, 0.0f);
    }
}
// Vectors per thread the resident kernels are built for, and whether a shape takes that path:
// the channel slice must fit, and there must be enough channels to occupy the machine.  (Measured
// with 24 vectors per thread: the registers spill and 128 workgroups of 16x128x76^2 are slower than
// the three launches; with a third of them in LDS they do not.)
constexpr int kResidentVectors = 8;
// the large form (128-bit vectors only): 16 vectors in registers + 8 in LDS (128 KB of the CU's 160)
constexpr int kResidentLargeRegs = 16, kResidentLargeLds = 8;
constexpr size_t kResidentLargeLdsBytes = static_cast<size_t>(kResidentLargeLds) * kResidentThreads * 16;

int resident_vectors(int batch, int channels, int spatial, bool vec)
{
    if (channels < 96) return 0;
    const size_t per_channel = static_cast<size_t>(batch) * spatial;
    const size_t vectors = (per_channel + (vec ? 3 : 0)) / (vec ? 4 : 1);
    const size_t per_thread = (vectors + kResidentThreads - 1) / kResidentThreads;
    if (per_thread <= kResidentVectors) return kResidentVectors;
    if (vec && per_thread <= kResidentLargeRegs + kResidentLargeLds) return kResidentLargeRegs + kResidentLargeLds;
    return 0;
}

// The scalar form with workgroups of kResidentNarrowThreads (twice the values per thread): when the full
// workgroups would outnumber the two places a compute unit has for them.  Measured at 16 x 1024 x 19^2:
// forward 14.6 against 16.3 us, backward 23.1 against 26.5; at 512 channels the forward gains 5 %, the
// backward loses 20 %.
constexpr int kResidentNarrowVectors = 2 * kResidentVectors;
bool resident_narrow(int batch, int channels, int spatial, bool vec, bool backward)
{
    if (vec || channels < (backward ? 1024 : 512)) return false;
    const size_t per_channel = static_cast<size_t>(batch) * spatial;
    return (per_channel + kResidentNarrowThreads - 1) / kResidentNarrowThreads <= kResidentNarrowVectors &&
           resident_vectors(batch, channels, spatial, vec) == kResidentVectors;
}

// A kernel that asks for more than 64 KB of dynamic LDS has to be allowed to, once.
int allow_large_lds(const void* kernel)
{
    static std::mutex mutex;
    static std::vector<const void*> allowed;
    std::lock_guard<std::mutex> lock(mutex);
    for (const void* k: allowed)
        if (k == kernel) return PXH_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(kResidentLargeLdsBytes));
    if (e != hipSuccess) {
        set_error("hipFuncSetAttribute(max dynamic LDS %zu): %s", kResidentLargeLdsBytes, hipGetErrorString(e));
        return static_cast<int>(e);
    }
    allowed.push_back(kernel);
    return PXH_OK;
}

ResidentGeom resident_geom(int batch, int channels, int spatial)
{
    return ResidentGeom{ channels, spatial, static_cast<uint32_t>(batch) * static_cast<uint32_t>(spatial),
                         FastDiv(static_cast<uint32_t>(spatial)) };
}

// workspace: [partial sums][per-channel constants]
size_t partial_bytes(int batch, int channels, int spatial)
{
    const ReduceGeom g = make_geom(batch, channels, spatial);
    const size_t b = static_cast<size_t>(channels) * g.blocks * sizeof(double2);
    return (b + 255) & ~static_cast<size_t>(255);
}

size_t workspace_bytes(int batch, int channels, int spatial)
{
    return partial_bytes(batch, channels, spatial) + static_cast<size_t>(channels) * sizeof(DxCoef);
}

void* coef_region(void* ws, int batch, int channels, int spatial)
{
    return static_cast<char*>(ws) + partial_bytes(batch, channels, spatial);
}

// The clipped backward: [partial sums][per-channel constants][norm partials][plan] for the three
// launches, [per-channel norm figures][per-channel sums][per-channel flags][plan] for the one-launch form.
constexpr size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }

struct ClippedRegions {
    double2* partial;
    DxCoef* coef;
    double2* norm_partial;
    double2* channel_norm;
    double2* channel_sums;
    int* channel_done;
    ClipPlan* plan;
};

size_t clipped_workspace_bytes(int batch, int channels, int spatial)
{
    const size_t c = static_cast<size_t>(channels);
    const size_t three = 2 * partial_bytes(batch, channels, spatial) + align256(c * sizeof(DxCoef)) + 256;
    const size_t one = 2 * align256(c * sizeof(double2)) + align256(c * sizeof(int)) + 256;
    return three > one ? three : one;
}

ClippedRegions clipped_regions(void* ws, int batch, int channels, int spatial)
{
    const size_t c = static_cast<size_t>(channels);
    char* base = static_cast<char*>(ws);
    ClippedRegions r;
    r.partial = reinterpret_cast<double2*>(base);
    r.coef = reinterpret_cast<DxCoef*>(base + partial_bytes(batch, channels, spatial));
    r.norm_partial = reinterpret_cast<double2*>(reinterpret_cast<char*>(r.coef) + align256(c * sizeof(DxCoef)));
    r.channel_norm = reinterpret_cast<double2*>(base);
    r.channel_sums = reinterpret_cast<double2*>(base + align256(c * sizeof(double2)));
    r.channel_done = reinterpret_cast<int*>(base + 2 * align256(c * sizeof(double2)));
    r.plan = reinterpret_cast<ClipPlan*>(base + clipped_workspace_bytes(batch, channels, spatial) - 256);
    return r;
}

// A tensor this large cannot stay in the last-level cache between two passes over it.
bool streams_past_cache(uint32_t total, int tensors)
{
    return static_cast<size_t>(total) * 4 * tensors >= kStreamingBytes;
}

int launch_stats(const float* x, float* mean, float* var, float* rolling_mean, float* rolling_var, const float* scale,
                 const float* bias, FoldCoef* table, int batch, int channels, int spatial, uint32_t total, void* ws,
                 hipStream_t stream)
{
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    const bool nt = streams_past_cache(total, 1);
    if (spatial % 4 == 0 && aligned16(x)) {
        if (nt) hipLaunchKernelGGL((bn_stats_partial_kernel<4, true>), grid, dim3(kBlock), 0, stream, x, g, partial);
        else hipLaunchKernelGGL((bn_stats_partial_kernel<4, false>), grid, dim3(kBlock), 0, stream, x, g, partial);
    } else {
        hipLaunchKernelGGL((bn_stats_partial_kernel<1, false>), grid, dim3(kBlock), 0, stream, x, g, partial);
    }
    int rc = check_launch("bn_stats_partial");
    if (rc) return rc;
    hipLaunchKernelGGL(bn_stats_finish_kernel, dim3(grid_for(channels, kBlock / kWave)), dim3(kBlock), 0, stream, x,
                       partial, channels, spatial, g.blocks, static_cast<double>(batch) * spatial, mean, var,
                       rolling_mean, rolling_var, scale, bias, table);
    return check_launch("bn_stats_finish");
}

// The linear shortcut taken into a forward pass (from == nullptr: none).
struct Residual {
    const float* from = nullptr;
    float alpha = 1.0f, beta = 1.0f;
};

// BN training forward + activation.  `get_workspace(need, &ws)` is asked for the `need` bytes of the
// three-launch form only when the shape does not take the one-launch form, which uses none.
template<typename GetWorkspace>
int bn_train_forward(const char* who, const float* x, float* y, float* pre_activation, float* x_saved, float* x_norm,
                     float* mean, float* var, float* rolling_mean, float* rolling_var, const float* scale,
                     const float* bias, int batch, int channels, int spatial, int activation,
                     GetWorkspace&& get_workspace, void* stream, const Residual& res = Residual{})
{
    if (!x || !y || !mean || !var || !rolling_mean || !rolling_var || !scale || !bias)
        return fail_invalid("%s: null pointer", who);
    if (x_saved == x) return fail_invalid("%s: x_saved must not alias x", who);
    EpilogueArgs a{};
    int rc = check_shape(who, batch, channels, spatial, &a.total);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    {
        const bool vec = spatial % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(pre_activation) &&
                         aligned16(x_saved) && aligned16(x_norm) && aligned16(res.from);
        const int per_thread = resident_vectors(batch, channels, spatial, vec);
        if (per_thread) {
            const ResidentFwdArgs r{ x, y, pre_activation, x_saved, x_norm, mean, var, rolling_mean, rolling_var,
                                     scale, bias, resident_geom(batch, channels, spatial), res.from, res.alpha, res.beta };
            // (with the shortcut's source on top, sixteen values per lane no longer fit the registers of four
            // workgroups per compute unit: that form keeps the full workgroups)
            const bool narrow = !res.from && resident_narrow(batch, channels, spatial, vec, false);
            const dim3 grid(channels), block(narrow ? kResidentNarrowThreads : kResidentThreads);
            int large_lds_rc = PXH_OK;
            const auto launch = [&]<int ACT, bool RES>() {
                constexpr int kT = kResidentThreads;
                if constexpr (!RES) {
                    if (narrow) {
                        hipLaunchKernelGGL((bn_resident_fwd_kernel<ACT, 1, kResidentNarrowVectors, 0, kResidentNarrowThreads>),
                                           grid, block, 0, s, r);
                        return;
                    }
                }
                if constexpr (RES) {
                    // The 128-bit form with the shortcut's source on top of eight vectors of the slice spills at
                    // 64 registers: half-size workgroups with twice the vectors per lane and twice the registers
                    // keep the same two workgroups per compute unit (16 x 512 x 38^2: 26.2 against 30.9 us).
                    if (vec && per_thread <= kResidentVectors) {
                        const size_t vectors = (static_cast<size_t>(batch) * spatial + 3) / 4;
                        const dim3 half(kResidentNarrowThreads);
                        if (vectors <= 12u * kResidentNarrowThreads)
                            hipLaunchKernelGGL((bn_resident_fwd_kernel<ACT, 4, 12, 0, kResidentNarrowThreads, true>), grid,
                                               half, 0, s, r);
                        else
                            hipLaunchKernelGGL((bn_resident_fwd_kernel<ACT, 4, 16, 0, kResidentNarrowThreads, true>), grid,
                                               half, 0, s, r);
                        return;
                    }
                }
                if (per_thread > kResidentVectors) {
                    auto kernel = bn_resident_fwd_kernel<ACT, 4, kResidentLargeRegs, kResidentLargeLds, kT, RES>;
                    large_lds_rc = allow_large_lds(reinterpret_cast<const void*>(kernel));
                    if (large_lds_rc == PXH_OK)
                        hipLaunchKernelGGL(kernel, grid, block, kResidentLargeLdsBytes, s, r);
                } else if (vec) {
                    hipLaunchKernelGGL((bn_resident_fwd_kernel<ACT, 4, kResidentVectors, 0, kT, RES>), grid, block, 0, s, r);
                } else {
                    hipLaunchKernelGGL((bn_resident_fwd_kernel<ACT, 1, kResidentVectors, 0, kT, RES>), grid, block, 0, s, r);
                }
            };
            const bool known = dispatch_activation(activation, [&]<int ACT>() {
                if (res.from) launch.template operator()<ACT, true>();
                else launch.template operator()<ACT, false>();
            });
            if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
            if (large_lds_rc) return large_lds_rc;
            return check_launch(who);
        }
    }
    void* ws;
    rc = get_workspace(workspace_bytes(batch, channels, spatial), &ws);
    if (rc) return rc;
    FoldCoef* table = static_cast<FoldCoef*>(coef_region(ws, batch, channels, spatial));
    rc = launch_stats(x, mean, var, rolling_mean, rolling_var, scale, bias, table, batch, channels, spatial, a.total,
                      ws, s);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation; a.x_saved = x_saved; a.x_norm = x_norm;
    a.table = table;
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    a.residual = res.from; a.res_alpha = res.alpha; a.res_beta = res.beta;
    return launch_epilogue_fwd<true>(who, a, activation, s);
}

}  // namespace
}  // namespace pxh

using namespace pxh;

extern "C" {

size_t pxh_bn_workspace_bytes(int batch, int channels, int spatial)
{
    if (batch <= 0 || channels <= 0 || spatial <= 0) return 0;
    return workspace_bytes(batch, channels, spatial);
}

size_t pxh_bn_folded_bytes(int channels)
{
    return channels > 0 ? static_cast<size_t>(channels) * sizeof(FoldCoef) : 0;
}

int pxh_bn_fold(const float* rolling_mean, const float* rolling_var, const float* scale, const float* bias,
                int channels, void* folded, void* stream)
{
    if (!rolling_mean || !rolling_var || !scale || !bias || !folded) return fail_invalid("pxh_bn_fold: null pointer");
    if (channels <= 0) return fail_invalid("pxh_bn_fold: channels must be positive");
    if (!aligned16(folded)) return fail_invalid("pxh_bn_fold: folded must be 16-byte aligned");
    hipLaunchKernelGGL(bn_fold_kernel, dim3(grid_for(channels, kBlock)), dim3(kBlock), 0, as_stream(stream),
                       rolling_mean, rolling_var, scale, bias, channels, static_cast<FoldCoef*>(folded));
    return check_launch("pxh_bn_fold");
}

int pxh_bn_folded_act_forward(const float* x, float* y, float* pre_activation, const void* folded, int batch,
                              int channels, int spatial, int activation, void* stream)
{
    if (!x || !y || !folded) return fail_invalid("pxh_bn_folded_act_forward: null pointer");
    if (!aligned16(folded)) return fail_invalid("pxh_bn_folded_act_forward: folded must be 16-byte aligned");
    EpilogueArgs a{};
    int rc = check_shape("pxh_bn_folded_act_forward", batch, channels, spatial, &a.total);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation;
    a.table = static_cast<const FoldCoef*>(folded);
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    return launch_epilogue_fwd<true>("pxh_bn_folded_act_forward", a, activation, as_stream(stream));
}

int pxh_bn_infer_act_forward(const float* x, float* y, float* pre_activation, const float* rolling_mean,
                             const float* rolling_var, const float* scale, const float* bias, int batch,
                             int channels, int spatial, int activation, void* workspace,
                             size_t workspace_bytes_given, void* stream)
{
    if (!x || !y || !rolling_mean || !rolling_var || !scale || !bias)
        return fail_invalid("pxh_bn_infer_act_forward: null pointer");
    uint32_t total;
    int rc = check_shape("pxh_bn_infer_act_forward", batch, channels, spatial, &total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, pxh_bn_folded_bytes(channels), &ws, as_stream(stream));
    if (rc) return rc;
    rc = pxh_bn_fold(rolling_mean, rolling_var, scale, bias, channels, ws, stream);
    if (rc) return rc;
    return pxh_bn_folded_act_forward(x, y, pre_activation, ws, batch, channels, spatial, activation, stream);
}

int pxh_bias_act_forward(const float* x, float* y, float* pre_activation, const float* bias, int batch,
                         int channels, int spatial, int activation, void* stream)
{
    if (!x || !y || !bias) return fail_invalid("pxh_bias_act_forward: null pointer");
    EpilogueArgs a{};
    int rc = check_shape("pxh_bias_act_forward", batch, channels, spatial, &a.total);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation; a.bias = bias;
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    return launch_epilogue_fwd<false>("pxh_bias_act_forward", a, activation, as_stream(stream));
}

int pxh_add_bias(float* output, const float* bias, int batch, int n, int size, void* stream)
{
    return pxh_bias_act_forward(output, output, nullptr, bias, batch, n, size, PXH_LINEAR, stream);
}

int pxh_bn_stats(const float* x, float* mean, float* var, int batch, int channels, int spatial, void* workspace,
                 size_t workspace_bytes_given, void* stream)
{
    if (!x || !mean || !var) return fail_invalid("pxh_bn_stats: null pointer");
    uint32_t total;
    int rc = check_shape("pxh_bn_stats", batch, channels, spatial, &total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws, as_stream(stream));
    if (rc) return rc;
    return launch_stats(x, mean, var, nullptr, nullptr, nullptr, nullptr, nullptr, batch, channels, spatial, total,
                        ws, as_stream(stream));
}

int pxh_bn_train_act_forward(const float* x, float* y, float* pre_activation, float* x_saved, float* x_norm,
                             float* mean, float* var, float* rolling_mean, float* rolling_var, const float* scale,
                             const float* bias, int batch, int channels, int spatial, int activation,
                             void* workspace, size_t workspace_bytes_given, void* stream)
{
    return bn_train_forward(
        "pxh_bn_train_act_forward", x, y, pre_activation, x_saved, x_norm, mean, var, rolling_mean, rolling_var,
        scale, bias, batch, channels, spatial, activation,
        [&](size_t need, void** ws) { return resolve_workspace(workspace, workspace_bytes_given, need, ws, as_stream(stream)); }, stream);
}

int pxh_bn_train_act_shortcut_forward(const float* x, float* y, float* pre_activation, float* x_saved, float* x_norm,
                                      float* mean, float* var, float* rolling_mean, float* rolling_var,
                                      const float* scale, const float* bias, const float* from, float alpha, float beta,
                                      int batch, int channels, int spatial, int activation, void* workspace,
                                      size_t workspace_bytes_given, void* stream)
{
    const char* who = "pxh_bn_train_act_shortcut_forward";
    if (!from) return fail_invalid("%s: null pointer (from)", who);
    if (from == x_saved || from == x_norm || from == pre_activation)
        return fail_invalid("%s: from must not alias an output other than y", who);
    return bn_train_forward(
        who, x, y, pre_activation, x_saved, x_norm, mean, var, rolling_mean, rolling_var, scale, bias, batch, channels,
        spatial, activation,
        [&](size_t need, void** ws) { return resolve_workspace(workspace, workspace_bytes_given, need, ws, as_stream(stream)); },
        stream, Residual{ from, alpha, beta });
}

int pxh_bn_folded_act_shortcut_forward(const float* x, float* y, float* pre_activation, const void* folded,
                                       const float* from, float alpha, float beta, int batch, int channels,
                                       int spatial, int activation, void* stream)
{
    const char* who = "pxh_bn_folded_act_shortcut_forward";
    if (!x || !y || !folded || !from) return fail_invalid("%s: null pointer", who);
    if (!aligned16(folded)) return fail_invalid("%s: folded must be 16-byte aligned", who);
    if (from == pre_activation) return fail_invalid("%s: from must not alias an output other than y", who);
    EpilogueArgs a{};
    int rc = check_shape(who, batch, channels, spatial, &a.total);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation;
    a.table = static_cast<const FoldCoef*>(folded);
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    a.residual = from; a.res_alpha = alpha; a.res_beta = beta;
    return launch_epilogue_fwd<true>(who, a, activation, as_stream(stream));
}

int pxh_bn_folded_act_maxpool_forward(const float* x, float* y, float* pooled, const void* folded, int batch,
                                      int channels, int height, int width, int activation, void* stream)
{
    const char* who = "pxh_bn_folded_act_maxpool_forward";
    if (!x || !pooled || !folded) return fail_invalid("%s: null pointer", who);
    if (!aligned16(folded)) return fail_invalid("%s: folded must be 16-byte aligned", who);
    if (height <= 0 || width <= 0) return fail_invalid("%s: height and width must be positive", who);
    if (pooled == x || pooled == y) return fail_invalid("%s: the pooled output must be a tensor of its own", who);
    uint32_t total;
    int rc = check_shape(who, batch, channels, height * width, &total);
    if (rc) return rc;
    if (height % 2 || width % 2 || !aligned16(x) || !aligned16(y) || !aligned16(pooled)) {
        set_error("%s: windows that do not tile the plane (%d x %d) or tensors off a 16-byte boundary take the two "
                  "calls (pxh_bn_folded_act_forward, pxh_maxpool_forward)", who, height, width);
        return PXH_ERR_UNSUPPORTED;
    }
    const uint32_t oh = height / 2, ow = width / 2;
    EpiloguePoolArgs a{};
    a.x = x; a.y = y; a.pooled = pooled;
    a.table = static_cast<const FoldCoef*>(folded);
    a.iw = width; a.ow = ow;
    a.by_oh = FastDiv(oh); a.by_channels = FastDiv(channels);
    const uint32_t outputs = total / 4;
    // x in, the pooled quarter out, the layer's own output when asked for
    const bool nt = static_cast<size_t>(total) * (y ? 9 : 5) >= kStreamingBytes;
    hipStream_t s = as_stream(stream);
    const auto launch = [&]<int ACT, int VX>() {
        a.units = outputs / VX;
        a.by_owv = FastDiv(ow / VX);
        const dim3 grid(grid_for(a.units, kBlock));
        if (nt) hipLaunchKernelGGL((epilogue_pool2_fwd_kernel<ACT, VX, true>), grid, dim3(kBlock), 0, s, a);
        else hipLaunchKernelGGL((epilogue_pool2_fwd_kernel<ACT, VX, false>), grid, dim3(kBlock), 0, s, a);
    };
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (width % 8 == 0) launch.template operator()<ACT, 4>();
        else if (width % 4 == 0) launch.template operator()<ACT, 2>();
        else launch.template operator()<ACT, 1>();
    });
    if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
    return check_launch(who);
}

int pxh_bn_train_act_forward_static(const float* x, float* y, float* pre_activation, float* x_saved, float* x_norm,
                                    float* mean, float* var, float* rolling_mean, float* rolling_var,
                                    const float* scale, const float* bias, int batch, int channels, int spatial,
                                    int activation, void* stream)
{
    const char* who = "pxh_bn_train_act_forward_static";
    return bn_train_forward(
        who, x, y, pre_activation, x_saved, x_norm, mean, var, rolling_mean, rolling_var, scale, bias, batch,
        channels, spatial, activation,
        [&](size_t need, void** ws) {
            if (need > kStaticScratchBytes) {
                set_error("%s: batch %d x channels %d x spatial %d needs %zu bytes of scratch, the built-in buffer "
                          "holds %zu; use pxh_bn_train_act_forward with a workspace of pxh_bn_workspace_bytes()",
                          who, batch, channels, spatial, need, kStaticScratchBytes);
                return PXH_ERR_WORKSPACE;
            }
            return static_scratch(who, ws);
        },
        stream);
}

// The rescale + clip in front of a backward, or none.
struct ClipSpec {
    bool on;
    float threshold, clip;
    float* norm_out;
};

static int bn_backward(const char* who, float* delta, const float* x, const float* pre_activation, const float* mean,
                       const float* var, const float* scale, const float* bias, float* scale_updates,
                       float* bias_updates, float* mean_delta, float* var_delta, int batch, int channels, int spatial,
                       int activation, const ClipSpec& cs, void* workspace, size_t workspace_bytes_given, void* stream)
{
    if (!delta || !x || !mean || !var || !scale || !bias || !scale_updates || !bias_updates)
        return fail_invalid("%s: null pointer", who);
    uint32_t total;
    int rc = check_shape(who, batch, channels, spatial, &total);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const bool rvec = spatial % 4 == 0 && aligned16(delta) && aligned16(x) && aligned16(pre_activation);
    const int per_thread = resident_vectors(batch, channels, spatial, rvec);
    void* ws = nullptr;
    ClippedRegions region{};
    ClipArgs clip{};
    if (cs.on) {
        rc = resolve_workspace(workspace, workspace_bytes_given, clipped_workspace_bytes(batch, channels, spatial), &ws, s);
        if (rc) return rc;
        region = clipped_regions(ws, batch, channels, spatial);
        clip = ClipArgs{ region.norm_partial, region.plan, cs.threshold, cs.clip, cs.norm_out };
    }
    if (per_thread) {
        const ResidentBwdArgs r{ BackwardArgs{ delta, x, pre_activation, mean, var, scale, bias }, scale_updates,
                                 bias_updates, mean_delta, var_delta, resident_geom(batch, channels, spatial),
                                 region.channel_norm, region.channel_sums, region.channel_done, clip };
        const bool narrow = resident_narrow(batch, channels, spatial, rvec, true);
        const dim3 block(narrow ? kResidentNarrowThreads : kResidentThreads);
        int large_lds_rc = PXH_OK;
        const auto launch = [&]<int ACT, int MODE>() {
            // the launch that follows the plan: one workgroup per compute unit at most, each walks channels
            const bool walks = MODE == kRedo && per_thread <= kResidentVectors && channels > kRedoWorkgroups;
            const dim3 grid(walks ? kRedoWorkgroups : channels);
            if (narrow) {
                hipLaunchKernelGGL((bn_resident_bwd_kernel<ACT, 1, kResidentNarrowVectors, 0, MODE, kResidentNarrowThreads>),
                                   grid, block, 0, s, r);
            } else if (per_thread > kResidentVectors) {
                auto kernel = bn_resident_bwd_kernel<ACT, 4, kResidentLargeRegs, kResidentLargeLds, MODE>;
                large_lds_rc = allow_large_lds(reinterpret_cast<const void*>(kernel));
                if (large_lds_rc == PXH_OK) hipLaunchKernelGGL(kernel, grid, block, kResidentLargeLdsBytes, s, r);
            } else if (rvec) {
                hipLaunchKernelGGL((bn_resident_bwd_kernel<ACT, 4, kResidentVectors, 0, MODE>), grid, block, 0, s, r);
            } else {
                hipLaunchKernelGGL((bn_resident_bwd_kernel<ACT, 1, kResidentVectors, 0, MODE>), grid, block, 0, s, r);
            }
        };
        const bool known = dispatch_activation(activation, [&]<int ACT>() {
            if (!cs.on) {
                launch.template operator()<ACT, kPlain>();
            } else {
                launch.template operator()<ACT, kFirst>();
                if (large_lds_rc == PXH_OK) launch.template operator()<ACT, kRedo>();
            }
        });
        if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
        if (large_lds_rc) return large_lds_rc;
        return check_launch(who);
    }
    if (!cs.on) {
        rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws, s);
        if (rc) return rc;
    }
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    DxCoef* coef = static_cast<DxCoef*>(coef_region(ws, batch, channels, spatial));

    BackwardArgs b{ delta, x, pre_activation, mean, var, scale, bias };
    const bool vec = rvec;
    const int tensors = pre_activation ? 3 : 2;
    const bool nt = vec && streams_past_cache(total, tensors);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    const dim3 finish_grid(grid_for(channels, kBlock / kWave));
    const auto sums = [&]<int ACT, int MODE>() {
        if (nt) {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, true, false, 4, true, MODE>), grid, dim3(kBlock), 0, s, b, g,
                               partial, clip);
        } else if (vec) {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, true, false, 4, false, MODE>), grid, dim3(kBlock), 0, s, b, g,
                               partial, clip);
        } else {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, true, false, 1, false, MODE>), grid, dim3(kBlock), 0, s, b, g,
                               partial, clip);
        }
    };
    const auto finish = [&]<int MODE>() {
        if constexpr (MODE == kFirst)
            hipLaunchKernelGGL((bwd_finish_kernel<true, MODE, kPlanThreads>), dim3(grid_for(channels, kPlanThreads / kWave)),
                               dim3(kPlanThreads), 0, s, partial, channels, g.blocks, batch * spatial, mean, var, scale,
                               bias, scale_updates, bias_updates, mean_delta, var_delta, coef, clip);
        else
            hipLaunchKernelGGL((bwd_finish_kernel<true, MODE>), finish_grid, dim3(kBlock), 0, s, partial, channels,
                               g.blocks, batch * spatial, mean, var, scale, bias, scale_updates, bias_updates,
                               mean_delta, var_delta, coef, clip);
    };
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (!cs.on) {
            sums.template operator()<ACT, kPlain>();
        } else {
            sums.template operator()<ACT, kFirst>();
            finish.template operator()<kFirst>();
            sums.template operator()<ACT, kRedo>();
        }
    });
    if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
    rc = check_launch("bn_backward_partial");
    if (rc) return rc;
    if (cs.on) finish.template operator()<kRedo>();
    else finish.template operator()<kPlain>();
    rc = check_launch("bn_backward_finish");
    if (rc) return rc;

    DxArgs d{};
    d.delta = delta; d.x = x; d.pre = pre_activation; d.coef = coef;
    d.by_spatial = FastDiv(spatial); d.by_channels = FastDiv(channels); d.total = total;
    d.plan = cs.on ? region.plan : nullptr;
    const bool dx_vec = aligned16(delta) && aligned16(x) && aligned16(pre_activation);
    const bool dx_nt = streams_past_cache(total, tensors + 1);
    const auto dx = [&]<int ACT, bool CLIPPED>() {
        if (dx_vec) {
            const dim3 dx_grid(grid_for(total, static_cast<size_t>(kBlock) * 4));
            if (dx_nt) hipLaunchKernelGGL((bn_dx_kernel<ACT, true, CLIPPED>), dx_grid, dim3(kBlock), 0, s, d);
            else hipLaunchKernelGGL((bn_dx_kernel<ACT, false, CLIPPED>), dx_grid, dim3(kBlock), 0, s, d);
        } else {
            hipLaunchKernelGGL((bn_dx_scalar_kernel<ACT, CLIPPED>), dim3(grid_for(total, kBlock)), dim3(kBlock), 0, s, d);
        }
    };
    dispatch_activation(activation, [&]<int ACT>() {
        if (cs.on) dx.template operator()<ACT, true>();
        else dx.template operator()<ACT, false>();
    });
    return check_launch("bn_backward_dx");
}

int pxh_bn_act_backward(float* delta, const float* x, const float* pre_activation, const float* mean,
                        const float* var, const float* scale, const float* bias, float* scale_updates,
                        float* bias_updates, float* mean_delta, float* var_delta, int batch, int channels,
                        int spatial, int activation, void* workspace, size_t workspace_bytes_given, void* stream)
{
    return bn_backward("pxh_bn_act_backward", delta, x, pre_activation, mean, var, scale, bias, scale_updates,
                       bias_updates, mean_delta, var_delta, batch, channels, spatial, activation,
                       ClipSpec{ false, 0.0f, 0.0f, nullptr }, workspace, workspace_bytes_given, stream);
}

size_t pxh_bn_clipped_workspace_bytes(int batch, int channels, int spatial)
{
    if (batch <= 0 || channels <= 0 || spatial <= 0) return 0;
    return clipped_workspace_bytes(batch, channels, spatial);
}

int pxh_bn_act_backward_clipped(float* delta, const float* x, const float* pre_activation, const float* mean,
                                const float* var, const float* scale, const float* bias, float* scale_updates,
                                float* bias_updates, float* mean_delta, float* var_delta, int batch, int channels,
                                int spatial, int activation, float threshold, float clip, float* norm_out,
                                void* workspace, size_t workspace_bytes_given, void* stream)
{
    return bn_backward("pxh_bn_act_backward_clipped", delta, x, pre_activation, mean, var, scale, bias, scale_updates,
                       bias_updates, mean_delta, var_delta, batch, channels, spatial, activation,
                       ClipSpec{ true, threshold, clip, norm_out }, workspace, workspace_bytes_given, stream);
}

static int bias_backward(const char* who, float* delta, const float* pre_activation, float* bias_updates, int batch,
                         int channels, int spatial, int activation, const ClipSpec& cs, void* workspace,
                         size_t workspace_bytes_given, void* stream)
{
    if (!delta || !bias_updates) return fail_invalid("%s: null pointer", who);
    if (activation != PXH_LINEAR && !pre_activation)
        return fail_invalid("%s: pre_activation is required for a non-linear activation", who);
    uint32_t total;
    int rc = check_shape(who, batch, channels, spatial, &total);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given,
                           cs.on ? clipped_workspace_bytes(batch, channels, spatial)
                                 : workspace_bytes(batch, channels, spatial), &ws, s);
    if (rc) return rc;
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    ClipArgs clip{};
    if (cs.on) {
        const ClippedRegions region = clipped_regions(ws, batch, channels, spatial);
        clip = ClipArgs{ region.norm_partial, region.plan, cs.threshold, cs.clip, cs.norm_out };
    }
    BackwardArgs b{ delta, nullptr, pre_activation, nullptr, nullptr, nullptr, nullptr };
    const bool vec = spatial % 4 == 0 && aligned16(delta) && aligned16(pre_activation);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    const dim3 finish_grid(grid_for(channels, kBlock / kWave));
    const auto sums = [&]<int ACT, bool WRITE, int MODE>() {
        if (vec) {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, false, WRITE, 4, false, MODE>), grid, dim3(kBlock), 0, s, b, g,
                               partial, clip);
        } else {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, false, WRITE, 1, false, MODE>), grid, dim3(kBlock), 0, s, b, g,
                               partial, clip);
        }
    };
    const auto finish = [&]<int MODE>() {
        if constexpr (MODE == kFirst)
            hipLaunchKernelGGL((bwd_finish_kernel<false, MODE, kPlanThreads>), dim3(grid_for(channels, kPlanThreads / kWave)),
                               dim3(kPlanThreads), 0, s, partial, channels, g.blocks, batch * spatial, nullptr, nullptr,
                               nullptr, nullptr, nullptr, bias_updates, nullptr, nullptr, nullptr, clip);
        else
            hipLaunchKernelGGL((bwd_finish_kernel<false, MODE>), finish_grid, dim3(kBlock), 0, s, partial, channels,
                               g.blocks, batch * spatial, nullptr, nullptr, nullptr, nullptr, nullptr, bias_updates,
                               nullptr, nullptr, nullptr, clip);
    };
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (!cs.on) {
            sums.template operator()<ACT, true, kPlain>();
        } else {
            // the sums of the delta as it came (nothing written), the plan, then the pass that writes:
            // it leaves at once when nothing changes and the activation is linear
            sums.template operator()<ACT, false, kFirst>();
            finish.template operator()<kFirst>();
            sums.template operator()<ACT, true, kRedo>();
        }
    });
    if (!known) return fail_invalid("%s: unknown activation %d", who, activation);
    rc = check_launch("bias_backward_partial");
    if (rc) return rc;
    if (cs.on) finish.template operator()<kRedo>();
    else finish.template operator()<kPlain>();
    return check_launch("bias_backward_finish");
}

int pxh_bias_act_backward(float* delta, const float* pre_activation, float* bias_updates, int batch, int channels,
                          int spatial, int activation, void* workspace, size_t workspace_bytes_given, void* stream)
{
    return bias_backward("pxh_bias_act_backward", delta, pre_activation, bias_updates, batch, channels, spatial,
                         activation, ClipSpec{ false, 0.0f, 0.0f, nullptr }, workspace, workspace_bytes_given, stream);
}

int pxh_bias_act_backward_clipped(float* delta, const float* pre_activation, float* bias_updates, int batch,
                                  int channels, int spatial, int activation, float threshold, float clip,
                                  float* norm_out, void* workspace, size_t workspace_bytes_given, void* stream)
{
    return bias_backward("pxh_bias_act_backward_clipped", delta, pre_activation, bias_updates, batch, channels,
                         spatial, activation, ClipSpec{ true, threshold, clip, norm_out }, workspace,
                         workspace_bytes_given, stream);
}

int pxh_backward_bias(float* bias_updates, const float* delta, int batch, int n, int size, void* workspace,
                      size_t workspace_bytes_given, void* stream)
{
    // delta is only read on the linear path
    return pxh_bias_act_backward(const_cast<float*>(delta), nullptr, bias_updates, batch, n, size, PXH_LINEAR,
                                 workspace, workspace_bytes_given, stream);
}

}
