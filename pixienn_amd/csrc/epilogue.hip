// Conv-layer epilogue for gfx950: batch-norm (inference and training) + bias + activation,
// forward and backward, as one-pass NCHW streaming kernels and per-channel reductions.
//
// Numerics follow the CPU layer (src/BatchNorm.cpp, src/CpuUtil.cpp:248-342 of the reference):
//   x_hat = float( double(x - mean) / (sqrt(double(var)) + 1e-5f) )     eps OUTSIDE the root
//   pre   = float(float(x_hat * scale) + bias)                           two fp32 roundings
// The quotient is formed as double(x - mean) * (1 / denominator): the double product rounds to
// the same float as the double quotient except in ~1e-8 of cases.
#include "stream.h"

namespace pxh {
namespace {

constexpr float kEps = .00001f;
constexpr int kTable = 160;               // per-workgroup plane table entries
constexpr int kMinSpatialFast = 28;       // kChunk / 28 + 2 <= kTable

struct PlaneCoef {
    double rdenom;   // 1 / (sqrt(var) + eps)
    float mean, scale, bias, pad;
};

__device__ __forceinline__ PlaneCoef make_coef(const float* mean, const float* var, const float* scale,
                                               const float* bias, uint32_t c)
{
    PlaneCoef k;
    k.mean = mean[c];
    k.scale = scale[c];
    k.bias = bias[c];
    k.pad = 0.0f;
    k.rdenom = 1.0 / (sqrt(static_cast<double>(var[c])) + static_cast<double>(kEps));
    return k;
}

struct EpilogueArgs {
    const float* x;
    float* y;
    float* pre;        // nullable
    float* x_saved;    // nullable
    float* x_norm;     // nullable
    const float* mean;
    const float* var;
    const float* scale;
    const float* bias;
    FastDiv by_spatial;
    FastDiv by_channels;
    uint32_t total;
};

template<int ACT, bool BN>
__device__ __forceinline__ float epilogue_value(float x, const PlaneCoef& k, float& xn)
{
    float pre;
    if constexpr (BN) {
        const float t = x - k.mean;
        xn = static_cast<float>(static_cast<double>(t) * k.rdenom);
        const float s = xn * k.scale;
        pre = s + k.bias;
    } else {
        xn = 0.0f;
        pre = x + k.bias;
    }
    return pre;
}

// One workgroup streams kChunk consecutive elements; the (few) planes it touches get their
// per-channel constants computed once into LDS while the loads are in flight.
template<int ACT, bool BN>
__global__ __launch_bounds__(kBlock) void epilogue_fwd_kernel(EpilogueArgs a)
{
    __shared__ PlaneCoef tab[kTable];
    const uint32_t chunk0 = blockIdx.x * static_cast<uint32_t>(kChunk);
    const uint32_t hw = a.by_spatial.d;
    uint32_t first_plane, rem0;
    a.by_spatial.divmod(chunk0, first_plane, rem0);

    Pack<4> xin[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint32_t e = chunk0 + (u * kBlock + threadIdx.x) * 4;
        if (e + 3 < a.total) {
            xin[u] = ld<4>(a.x, e);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) xin[u].v[k] = (e + k < a.total) ? a.x[e + k] : 0.0f;
        }
    }

    const uint32_t chunk_end = min(chunk0 + static_cast<uint32_t>(kChunk), a.total);
    const uint32_t nplanes = a.by_spatial.div(chunk_end - 1) - first_plane + 1;
    if (threadIdx.x < nplanes) {
        uint32_t q, c;
        a.by_channels.divmod(first_plane + threadIdx.x, q, c);
        PlaneCoef k;
        if constexpr (BN) {
            k = make_coef(a.mean, a.var, a.scale, a.bias, c);
        } else {
            k.rdenom = 0.0;
            k.mean = 0.0f;
            k.scale = 1.0f;
            k.bias = a.bias[c];
            k.pad = 0.0f;
        }
        tab[threadIdx.x] = k;
    }
    __syncthreads();

#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint32_t l = (u * kBlock + threadIdx.x) * 4;
        const uint32_t e = chunk0 + l;
        if (e >= a.total) continue;
        uint32_t lp, r;
        a.by_spatial.divmod(rem0 + l, lp, r);
        Pack<4> yo, po, no;
        PlaneCoef k = tab[lp];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (r + j == hw) k = tab[lp + 1];
            po.v[j] = epilogue_value<ACT, BN>(xin[u].v[j], k, no.v[j]);
            yo.v[j] = act_apply<ACT>(po.v[j]);
        }
        if (e + 3 < a.total) {
            if (a.x_saved) st<4>(a.x_saved, e, xin[u]);
            if (BN && a.x_norm) st<4>(a.x_norm, e, no);
            if (a.pre) st<4>(a.pre, e, po);
            st<4>(a.y, e, yo);
        } else {
            for (int j = 0; j < 4 && e + j < a.total; ++j) {
                if (a.x_saved) a.x_saved[e + j] = xin[u].v[j];
                if (BN && a.x_norm) a.x_norm[e + j] = no.v[j];
                if (a.pre) a.pre[e + j] = po.v[j];
                a.y[e + j] = yo.v[j];
            }
        }
    }
}

// Any shape, any alignment: one element per lane, constants recomputed per element.
template<int ACT, bool BN>
__global__ __launch_bounds__(kBlock) void epilogue_fwd_generic_kernel(EpilogueArgs a)
{
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= a.total) return;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    PlaneCoef k;
    if constexpr (BN) {
        k = make_coef(a.mean, a.var, a.scale, a.bias, c);
    } else {
        k.bias = a.bias[c];
    }
    const float x = a.x[e];
    float xn;
    const float pre = epilogue_value<ACT, BN>(x, k, xn);
    if (a.x_saved) a.x_saved[e] = x;
    if (BN && a.x_norm) a.x_norm[e] = xn;
    if (a.pre) a.pre[e] = pre;
    a.y[e] = act_apply<ACT>(pre);
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
int launch_epilogue_fwd(const char* who, EpilogueArgs a, int spatial, int activation, hipStream_t stream)
{
    const bool fast = spatial >= kMinSpatialFast && aligned16(a.x) && aligned16(a.y) && aligned16(a.pre) &&
                      aligned16(a.x_saved) && aligned16(a.x_norm);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (fast) {
            hipLaunchKernelGGL((epilogue_fwd_kernel<ACT, BN>), dim3(grid_for(a.total, kChunk)), dim3(kBlock), 0,
                               stream, a);
        } else {
            hipLaunchKernelGGL((epilogue_fwd_generic_kernel<ACT, BN>), dim3(grid_for(a.total, kBlock)),
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
constexpr int kSeg = kWave * 4 * kUnroll;   // 1024 floats
constexpr int kItemsPerBlock = 16;

struct ReducePlan {
    int parts;    // segments per plane
    int items;    // batch * parts
    int blocks;   // workgroups per channel
};

ReducePlan make_plan(int batch, int spatial)
{
    ReducePlan p;
    p.parts = (spatial + kSeg - 1) / kSeg;
    p.items = batch * p.parts;
    p.blocks = (p.items + kItemsPerBlock - 1) / kItemsPerBlock;
    return p;
}

struct ReduceGeom {
    int channels, spatial, parts, items, blocks;
    FastDiv by_parts;
    FastDiv by_blocks;
};

ReduceGeom make_geom(int batch, int channels, int spatial)
{
    ReducePlan p = make_plan(batch, spatial);
    ReduceGeom g;
    g.channels = channels;
    g.spatial = spatial;
    g.parts = p.parts;
    g.items = p.items;
    g.blocks = p.blocks;
    g.by_parts = FastDiv(static_cast<uint32_t>(p.parts));
    g.by_blocks = FastDiv(static_cast<uint32_t>(p.blocks));
    return g;
}

// Visits every element of this workgroup's items: f(value_index, lane_local_count) is called as
// body(offset_in_tensor) for V consecutive floats.  Returns through the functor's own state.
template<int V, typename Body>
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
template<int V>
__global__ __launch_bounds__(kBlock) void bn_stats_partial_kernel(const float* x, ReduceGeom g, double2* partial)
{
    __shared__ double slots[2][kBlock / kWave];
    uint32_t c, j;
    g.by_blocks.divmod(blockIdx.x, c, j);
    const float shift = x[static_cast<size_t>(c) * g.spatial];
    double s1 = 0.0, s2 = 0.0;
    for_each_item<V>(g, c, j, [&](size_t base, int seg0, int seg1, int lane) {
        constexpr int kLoads = kSeg / (kWave * V);
        Pack<V> v[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) v[u] = ld<V>(x, base + off);
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

// One wavefront per channel adds the channel's partials and finishes mean / variance.
__global__ __launch_bounds__(kBlock) void bn_stats_finish_kernel(const float* x, const double2* partial, int channels,
                                                                 int spatial, int blocks, double count, float* mean,
                                                                 float* var, float* rolling_mean, float* rolling_var)
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
        const double shift = static_cast<double>(x[static_cast<size_t>(c) * spatial]);
        const double m = s1 / count;
        double v = (s2 - s1 * m) / count;
        if (v < 0.0) v = 0.0;
        const float fm = static_cast<float>(shift + m);
        const float fv = static_cast<float>(v);
        mean[c] = fm;
        var[c] = fv;
        if (rolling_mean) {
            // sscal then saxpy: two fp32 roundings each (src/BatchNorm.cpp:53-56)
            float r = 0.99f * rolling_mean[c];
            rolling_mean[c] = r + .01f * fm;
            r = 0.99f * rolling_var[c];
            rolling_var[c] = r + .01f * fv;
        }
    }
}

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

template<int ACT, bool BN, bool WRITE, int V>
__global__ __launch_bounds__(kBlock) void bwd_partial_kernel(BackwardArgs a, ReduceGeom g, double2* partial)
{
    __shared__ double slots[2][kBlock / kWave];
    uint32_t c, j;
    g.by_blocks.divmod(blockIdx.x, c, j);
    PlaneCoef k;
    if constexpr (BN) k = make_coef(a.mean, a.var, a.scale, a.bias, c);
    const bool recompute = BN && a.pre == nullptr;
    double sa = 0.0, sb = 0.0;
    for_each_item<V>(g, c, j, [&](size_t base, int seg0, int seg1, int lane) {
        constexpr int kLoads = kSeg / (kWave * V);
        Pack<V> d[kLoads], xv[kLoads], pv[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) {
                d[u] = ld<V>(a.delta, base + off);
                if constexpr (BN) xv[u] = ld<V>(a.x, base + off);
                if constexpr (ACT != PXH_LINEAR) {
                    if (!recompute) pv[u] = ld<V>(a.pre, base + off);
                }
            }
        }
        float fa = 0.0f, fb = 0.0f;
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int off = seg0 + (u * kWave + lane) * V;
            if (off < seg1) {
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    float dv = d[u].v[q];
                    if constexpr (ACT != PXH_LINEAR) {
                        float pre;
                        if (recompute) {
                            float xn;
                            pre = epilogue_value<ACT, true>(xv[u].v[q], k, xn);
                        } else {
                            pre = pv[u].v[q];
                        }
                        dv = dv * act_grad<ACT>(pre);
                        d[u].v[q] = dv;
                    }
                    fa += dv;
                    if constexpr (BN) fb += dv * (xv[u].v[q] - k.mean);
                }
                if constexpr (WRITE && ACT != PXH_LINEAR) st<V>(a.delta, base + off, d[u]);
            }
        }
        sa += static_cast<double>(fa);
        sb += static_cast<double>(fb);
    });
    const double ta = block_sum(sa, slots[0]);
    const double tb = block_sum(sb, slots[1]);
    if (threadIdx.x == 0) partial[blockIdx.x] = make_double2(ta, tb);
}

// Per-channel constants of the dx pass, produced by the finish kernel.
struct BackwardCoef {
    double rroot;     // 1 / sqrt(float(var + eps))
    double c2;        // var_delta * 2 / count
    double md_term;   // float(mean_delta / float(count))
};

template<bool BN>
__global__ __launch_bounds__(kBlock) void bwd_finish_kernel(const double2* partial, int channels, int blocks, int count,
                                                            const float* var, const float* scale,
                                                            float* scale_updates, float* bias_updates,
                                                            float* mean_delta, float* var_delta, BackwardCoef* coef)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int c = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (c >= channels) return;
    double sa = 0.0, sb = 0.0;
    for (int j = lane; j < blocks; j += kWave) {
        const double2 p = partial[static_cast<size_t>(c) * blocks + j];
        sa += p.x;
        sb += p.y;
    }
    sa = wave_sum(sa);
    sb = wave_sum(sb);
    if (lane == 0) {
        bias_updates[c] += static_cast<float>(sa);
        if constexpr (BN) {
            const float v = var[c];
            const float s = scale[c];
            // sum d' * x_hat with x_hat = (x - mean) / (sqrt(var) + eps)
            const double denom = sqrt(static_cast<double>(v)) + static_cast<double>(kEps);
            scale_updates[c] += static_cast<float>(sb / denom);
            // sums of d'' = d' * scale
            const float sum_dd = static_cast<float>(sa * static_cast<double>(s));
            const float sum_ddx = static_cast<float>(sb * static_cast<double>(s));
            const float ve = v + kEps;
            const float md = static_cast<float>(static_cast<double>(sum_dd) * (-1. / static_cast<double>(sqrtf(ve))));
            const float vd = sum_ddx * (-.5f * powf(ve, -3.0f / 2.0f));
            if (mean_delta) mean_delta[c] = md;
            if (var_delta) var_delta[c] = vd;
            BackwardCoef k;
            k.rroot = 1.0 / sqrt(static_cast<double>(ve));
            k.c2 = static_cast<double>(vd) * 2. / static_cast<double>(count);
            k.md_term = static_cast<double>(md / static_cast<float>(count));
            coef[c] = k;
        }
    }
}

struct DxArgs {
    float* delta;
    const float* x;
    const float* pre;   // nullable: recomputed
    const float* mean;
    const float* var;
    const float* scale;
    const float* bias;
    const BackwardCoef* coef;
    FastDiv by_spatial;
    FastDiv by_channels;
    uint32_t total;
};

struct DxCoef {
    PlaneCoef f;
    BackwardCoef b;
};

template<int ACT>
__device__ __forceinline__ float dx_value(float d, float x, float pre_in, bool recompute, const DxCoef& k)
{
    if constexpr (ACT != PXH_LINEAR) {
        float pre = pre_in;
        if (recompute) {
            float xn;
            pre = epilogue_value<ACT, true>(x, k.f, xn);
        }
        d = d * act_grad<ACT>(pre);
    }
    const float dd = d * k.f.scale;
    const float xm = x - k.f.mean;
    // src/CpuUtil.cpp:336-338 evaluated in double, stored as float
    const double v = static_cast<double>(dd) * k.b.rroot + k.b.c2 * static_cast<double>(xm) + k.b.md_term;
    return static_cast<float>(v);
}

template<int ACT>
__global__ __launch_bounds__(kBlock) void bn_dx_kernel(DxArgs a)
{
    __shared__ DxCoef tab[kTable];
    const uint32_t chunk0 = blockIdx.x * static_cast<uint32_t>(kChunk);
    const uint32_t hw = a.by_spatial.d;
    uint32_t first_plane, rem0;
    a.by_spatial.divmod(chunk0, first_plane, rem0);
    const bool recompute = a.pre == nullptr;

    Pack<4> din[kUnroll], xin[kUnroll], pin[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint32_t e = chunk0 + (u * kBlock + threadIdx.x) * 4;
        if (e + 3 < a.total) {
            din[u] = ld<4>(a.delta, e);
            xin[u] = ld<4>(a.x, e);
            if (ACT != PXH_LINEAR && !recompute) pin[u] = ld<4>(a.pre, e);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const bool ok = e + k < a.total;
                din[u].v[k] = ok ? a.delta[e + k] : 0.0f;
                xin[u].v[k] = ok ? a.x[e + k] : 0.0f;
                pin[u].v[k] = (ok && ACT != PXH_LINEAR && !recompute) ? a.pre[e + k] : 0.0f;
            }
        }
    }

    const uint32_t chunk_end = min(chunk0 + static_cast<uint32_t>(kChunk), a.total);
    const uint32_t nplanes = a.by_spatial.div(chunk_end - 1) - first_plane + 1;
    if (threadIdx.x < nplanes) {
        uint32_t q, c;
        a.by_channels.divmod(first_plane + threadIdx.x, q, c);
        DxCoef k;
        k.f = make_coef(a.mean, a.var, a.scale, a.bias, c);
        k.b = a.coef[c];
        tab[threadIdx.x] = k;
    }
    __syncthreads();

#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const uint32_t l = (u * kBlock + threadIdx.x) * 4;
        const uint32_t e = chunk0 + l;
        if (e >= a.total) continue;
        uint32_t lp, r;
        a.by_spatial.divmod(rem0 + l, lp, r);
        Pack<4> out;
        if (r + 3 < hw) {
            const DxCoef k = tab[lp];
#pragma unroll
            for (int j = 0; j < 4; ++j) out.v[j] = dx_value<ACT>(din[u].v[j], xin[u].v[j], pin[u].v[j], recompute, k);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const DxCoef k = tab[lp + (r + j >= hw ? 1 : 0)];
                out.v[j] = dx_value<ACT>(din[u].v[j], xin[u].v[j], pin[u].v[j], recompute, k);
            }
        }
        if (e + 3 < a.total) {
            st<4>(a.delta, e, out);
        } else {
            for (int j = 0; j < 4 && e + j < a.total; ++j) a.delta[e + j] = out.v[j];
        }
    }
}

template<int ACT>
__global__ __launch_bounds__(kBlock) void bn_dx_generic_kernel(DxArgs a)
{
    const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= a.total) return;
    uint32_t plane, r, q, c;
    a.by_spatial.divmod(e, plane, r);
    a.by_channels.divmod(plane, q, c);
    DxCoef k;
    k.f = make_coef(a.mean, a.var, a.scale, a.bias, c);
    k.b = a.coef[c];
    const bool recompute = a.pre == nullptr;
    const float pre = (ACT != PXH_LINEAR && !recompute) ? a.pre[e] : 0.0f;
    a.delta[e] = dx_value<ACT>(a.delta[e], a.x[e], pre, recompute, k);
}

size_t partial_bytes(int batch, int channels, int spatial)
{
    const ReducePlan p = make_plan(batch, spatial);
    return static_cast<size_t>(channels) * p.blocks * sizeof(double2);
}

size_t workspace_bytes(int batch, int channels, int spatial)
{
    // partial sums, then the per-channel constants of the dx pass
    size_t b = partial_bytes(batch, channels, spatial);
    b = (b + 255) & ~static_cast<size_t>(255);
    return b + static_cast<size_t>(channels) * sizeof(BackwardCoef);
}

int launch_stats(const float* x, float* mean, float* var, float* rolling_mean, float* rolling_var, int batch,
                 int channels, int spatial, void* ws, hipStream_t stream)
{
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    if (spatial % 4 == 0 && aligned16(x)) {
        hipLaunchKernelGGL((bn_stats_partial_kernel<4>), grid, dim3(kBlock), 0, stream, x, g, partial);
    } else {
        hipLaunchKernelGGL((bn_stats_partial_kernel<1>), grid, dim3(kBlock), 0, stream, x, g, partial);
    }
    int rc = check_launch("bn_stats_partial");
    if (rc) return rc;
    hipLaunchKernelGGL(bn_stats_finish_kernel, dim3(grid_for(channels, kBlock / kWave)), dim3(kBlock), 0, stream, x,
                       partial, channels, spatial, g.blocks, static_cast<double>(batch) * spatial, mean, var,
                       rolling_mean, rolling_var);
    return check_launch("bn_stats_finish");
}

}  // namespace
}  // namespace pxh

using namespace pxh;

extern "C" {

int pxh_bn_infer_act_forward(const float* x, float* y, float* pre_activation, const float* rolling_mean,
                             const float* rolling_var, const float* scale, const float* bias, int batch,
                             int channels, int spatial, int activation, void* stream)
{
    if (!x || !y || !rolling_mean || !rolling_var || !scale || !bias)
        return fail_invalid("pxh_bn_infer_act_forward: null pointer");
    EpilogueArgs a{};
    int rc = check_shape("pxh_bn_infer_act_forward", batch, channels, spatial, &a.total);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation; a.x_saved = nullptr; a.x_norm = nullptr;
    a.mean = rolling_mean; a.var = rolling_var; a.scale = scale; a.bias = bias;
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    return launch_epilogue_fwd<true>("pxh_bn_infer_act_forward", a, spatial, activation, as_stream(stream));
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
    return launch_epilogue_fwd<false>("pxh_bias_act_forward", a, spatial, activation, as_stream(stream));
}

int pxh_add_bias(float* output, const float* bias, int batch, int n, int size, void* stream)
{
    return pxh_bias_act_forward(output, output, nullptr, bias, batch, n, size, PXH_LINEAR, stream);
}

size_t pxh_bn_workspace_bytes(int batch, int channels, int spatial)
{
    if (batch <= 0 || channels <= 0 || spatial <= 0) return 0;
    return workspace_bytes(batch, channels, spatial);
}

int pxh_bn_stats(const float* x, float* mean, float* var, int batch, int channels, int spatial, void* workspace,
                 size_t workspace_bytes_given, void* stream)
{
    if (!x || !mean || !var) return fail_invalid("pxh_bn_stats: null pointer");
    uint32_t total;
    int rc = check_shape("pxh_bn_stats", batch, channels, spatial, &total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws);
    if (rc) return rc;
    return launch_stats(x, mean, var, nullptr, nullptr, batch, channels, spatial, ws, as_stream(stream));
}

int pxh_bn_train_act_forward(const float* x, float* y, float* pre_activation, float* x_saved, float* x_norm,
                             float* mean, float* var, float* rolling_mean, float* rolling_var, const float* scale,
                             const float* bias, int batch, int channels, int spatial, int activation,
                             void* workspace, size_t workspace_bytes_given, void* stream)
{
    if (!x || !y || !mean || !var || !rolling_mean || !rolling_var || !scale || !bias)
        return fail_invalid("pxh_bn_train_act_forward: null pointer");
    if (x_saved == x) return fail_invalid("pxh_bn_train_act_forward: x_saved must not alias x");
    EpilogueArgs a{};
    int rc = check_shape("pxh_bn_train_act_forward", batch, channels, spatial, &a.total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    rc = launch_stats(x, mean, var, rolling_mean, rolling_var, batch, channels, spatial, ws, s);
    if (rc) return rc;
    a.x = x; a.y = y; a.pre = pre_activation; a.x_saved = x_saved; a.x_norm = x_norm;
    a.mean = mean; a.var = var; a.scale = scale; a.bias = bias;
    a.by_spatial = FastDiv(spatial); a.by_channels = FastDiv(channels);
    return launch_epilogue_fwd<true>("pxh_bn_train_act_forward", a, spatial, activation, s);
}

int pxh_bn_act_backward(float* delta, const float* x, const float* pre_activation, const float* mean,
                        const float* var, const float* scale, const float* bias, float* scale_updates,
                        float* bias_updates, float* mean_delta, float* var_delta, int batch, int channels,
                        int spatial, int activation, void* workspace, size_t workspace_bytes_given, void* stream)
{
    if (!delta || !x || !mean || !var || !scale || !bias || !scale_updates || !bias_updates)
        return fail_invalid("pxh_bn_act_backward: null pointer");
    uint32_t total;
    int rc = check_shape("pxh_bn_act_backward", batch, channels, spatial, &total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    size_t off = (partial_bytes(batch, channels, spatial) + 255) & ~static_cast<size_t>(255);
    BackwardCoef* coef = reinterpret_cast<BackwardCoef*>(static_cast<char*>(ws) + off);

    BackwardArgs b{ delta, x, pre_activation, mean, var, scale, bias };
    const bool vec = spatial % 4 == 0 && aligned16(delta) && aligned16(x) && aligned16(pre_activation);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (vec) {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, true, false, 4>), grid, dim3(kBlock), 0, s, b, g, partial);
        } else {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, true, false, 1>), grid, dim3(kBlock), 0, s, b, g, partial);
        }
    });
    if (!known) return fail_invalid("pxh_bn_act_backward: unknown activation %d", activation);
    rc = check_launch("bn_backward_partial");
    if (rc) return rc;
    hipLaunchKernelGGL((bwd_finish_kernel<true>), dim3(grid_for(channels, kBlock / kWave)), dim3(kBlock), 0, s, partial,
                       channels, g.blocks, batch * spatial, var, scale, scale_updates, bias_updates, mean_delta,
                       var_delta, coef);
    rc = check_launch("bn_backward_finish");
    if (rc) return rc;

    DxArgs d{};
    d.delta = delta; d.x = x; d.pre = pre_activation; d.mean = mean; d.var = var; d.scale = scale; d.bias = bias;
    d.coef = coef; d.by_spatial = FastDiv(spatial); d.by_channels = FastDiv(channels); d.total = total;
    const bool fast = spatial >= kMinSpatialFast && aligned16(delta) && aligned16(x) && aligned16(pre_activation);
    dispatch_activation(activation, [&]<int ACT>() {
        if (fast) {
            hipLaunchKernelGGL((bn_dx_kernel<ACT>), dim3(grid_for(total, kChunk)), dim3(kBlock), 0, s, d);
        } else {
            hipLaunchKernelGGL((bn_dx_generic_kernel<ACT>), dim3(grid_for(total, kBlock)), dim3(kBlock), 0, s, d);
        }
    });
    return check_launch("bn_backward_dx");
}

int pxh_bias_act_backward(float* delta, const float* pre_activation, float* bias_updates, int batch, int channels,
                          int spatial, int activation, void* workspace, size_t workspace_bytes_given, void* stream)
{
    if (!delta || !bias_updates) return fail_invalid("pxh_bias_act_backward: null pointer");
    if (activation != PXH_LINEAR && !pre_activation)
        return fail_invalid("pxh_bias_act_backward: pre_activation is required for a non-linear activation");
    uint32_t total;
    int rc = check_shape("pxh_bias_act_backward", batch, channels, spatial, &total);
    if (rc) return rc;
    void* ws;
    rc = resolve_workspace(workspace, workspace_bytes_given, workspace_bytes(batch, channels, spatial), &ws);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const ReduceGeom g = make_geom(batch, channels, spatial);
    double2* partial = static_cast<double2*>(ws);
    BackwardArgs b{ delta, nullptr, pre_activation, nullptr, nullptr, nullptr, nullptr };
    const bool vec = spatial % 4 == 0 && aligned16(delta) && aligned16(pre_activation);
    const dim3 grid(static_cast<unsigned>(channels) * g.blocks);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (vec) {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, false, true, 4>), grid, dim3(kBlock), 0, s, b, g, partial);
        } else {
            hipLaunchKernelGGL((bwd_partial_kernel<ACT, false, true, 1>), grid, dim3(kBlock), 0, s, b, g, partial);
        }
    });
    if (!known) return fail_invalid("pxh_bias_act_backward: unknown activation %d", activation);
    rc = check_launch("bias_backward_partial");
    if (rc) return rc;
    hipLaunchKernelGGL((bwd_finish_kernel<false>), dim3(grid_for(channels, kBlock / kWave)), dim3(kBlock), 0, s,
                       partial, channels, g.blocks, batch * spatial, nullptr, nullptr, nullptr, bias_updates, nullptr,
                       nullptr, nullptr);
    return check_launch("bias_backward_finish");
}

int pxh_backward_bias(float* bias_updates, const float* delta, int batch, int n, int size, void* workspace,
                      size_t workspace_bytes_given, void* stream)
{
    // delta is only read on the linear path
    return pxh_bias_act_backward(const_cast<float*>(delta), nullptr, bias_updates, batch, n, size, PXH_LINEAR,
                                 workspace, workspace_bytes_given, stream);
}

}
