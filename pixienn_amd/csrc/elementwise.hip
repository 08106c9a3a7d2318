// Flat fp32 streaming kernels: activation, fill/clip/multiply/axpy helpers, shortcut, Adam.
#include "stream.h"
#include "pixienn_hip_test.h"

#include <cmath>
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>

namespace pxh {
namespace {

// ---------------------------------------------------------------- activation
template<int ACT>
struct ActivateOp {
    float* x;
    template<int V> struct Regs { Pack<V> x; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const { r.x = ld<V, NT>(x, e); }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = act_apply<ACT>(r.x.v[k]);
        st<V, NT>(x, e, o);
    }
};

template<int ACT>
struct GradientOp {
    const float* x;
    float* delta;
    template<int V> struct Regs { Pack<V> x, d; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.x = ld<V, NT>(x, e);
        r.d = ld<V, NT>(delta, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = r.d.v[k] * act_grad<ACT>(r.x.v[k]);
        st<V, NT>(delta, e, o);
    }
};

// ---------------------------------------------------------------- helpers
// A fill writes a tensor nobody reads back soon (a cleared delta waits for the backward pass), so its
// stores go past the caches from a much smaller size on than the other kernels' (measured over the 107
// fills of a YOLOv3 forward pass: 0.14 ms of 4.96 less).
constexpr size_t kFillStreamingBytes = 8u << 20;

struct FillOp {
    float* x;
    float value;
    template<int V> struct Regs {};
    template<int V, bool NT> __device__ void load(size_t, Regs<V>&) const {}
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>&) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = value;
        st<V, NT>(x, e, o);
    }
};

struct ConstrainOp {
    float* x;
    float alpha;
    template<int V> struct Regs { Pack<V> x; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const { r.x = ld<V, NT>(x, e); }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = fminf(alpha, fmaxf(-alpha, r.x.v[k]));
        st<V, NT>(x, e, o);
    }
};

struct MulOp {
    const float* x;
    float* y;
    template<int V> struct Regs { Pack<V> x, y; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.x = ld<V, NT>(x, e);
        r.y = ld<V, NT>(y, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = r.x.v[k] * r.y.v[k];
        st<V, NT>(y, e, o);
    }
};

struct AxpyOp {
    const float* x;
    float* y;
    float alpha;
    template<int V> struct Regs { Pack<V> x, y; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.x = ld<V, NT>(x, e);
        r.y = ld<V, NT>(y, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const { finish_value<V, NT>(e, r); }
    // ... and returns what it left in y
    template<int V, bool NT> __device__ Pack<V> finish_value(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const float p = alpha * r.x.v[k];
            o.v[k] = r.y.v[k] + p;
        }
        st<V, NT>(y, e, o);
        return o;
    }
};

// ---------------------------------------------------------------- route (channel concat)
// One source layer of a concatenation: image b of the layer (layer_outputs floats, packed) sits
// at route + b*route_outputs + offset.  FORWARD copies layer -> route; BACKWARD adds the route
// slice into the layer's delta (x + y, one rounding, like saxpy with alpha = 1).
template<bool BACKWARD>
struct RouteOp {
    const float* src;      // forward: layer output; backward: route delta
    float* dst;            // forward: route output; backward: layer delta
    FastDiv by_image;      // layer_outputs
    uint32_t route_outputs, offset;
    template<int V> struct Regs { Pack<V> a, b; };
    __device__ __forceinline__ size_t concat_index(size_t e) const
    {
        uint32_t image, within;
        by_image.divmod(static_cast<uint32_t>(e), image, within);
        return static_cast<size_t>(image) * route_outputs + offset + within;
    }
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        if constexpr (BACKWARD) {
            r.a = ld<V, NT>(src, concat_index(e));
            r.b = ld<V, NT>(dst, e);
        } else {
            r.a = ld<V, NT>(src, e);
        }
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        if constexpr (BACKWARD) {
            Pack<V> o;
#pragma unroll
            for (int k = 0; k < V; ++k) o.v[k] = r.b.v[k] + r.a.v[k];
            st<V, NT>(dst, e, o);
        } else {
            st<V, NT>(dst, concat_index(e), r.a);
        }
    }
};

int check_route(const char* who, const void* a, const void* b, int batch, int layer_outputs, int route_outputs,
                int offset)
{
    if (batch < 0 || layer_outputs < 0 || route_outputs < 0 || offset < 0)
        return fail_invalid("%s: negative size", who);
    if (static_cast<int64_t>(offset) + layer_outputs > route_outputs)
        return fail_invalid("%s: slice [%d, %d) exceeds the %d outputs of the route", who, offset,
                            offset + layer_outputs, route_outputs);
    const int64_t n = static_cast<int64_t>(batch) * layer_outputs;
    if ((!a || !b) && n) return fail_invalid("%s: null pointer", who);
    if (n >= (int64_t(1) << 31) || static_cast<int64_t>(batch) * route_outputs >= (int64_t(1) << 31))
    {
        set_error("%s: tensors of 2^31 elements or more are not supported", who);
        return PXH_ERR_UNSUPPORTED;
    }
    return PXH_OK;
}

// ---------------------------------------------------------------- shortcut
// pre = alpha*in + beta*from (two products, one sum, each rounded); out = act(pre)
template<int ACT>
struct ShortcutForwardOp {
    const float* in;
    const float* from;
    float* out;
    float* pre;   // nullable
    float alpha, beta;
    template<int V> struct Regs { Pack<V> a, b; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.a = ld<V, NT>(in, e);
        r.b = ld<V, NT>(from, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> p, o;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const float pa = alpha * r.a.v[k];
            const float pb = beta * r.b.v[k];
            p.v[k] = pa + pb;
            o.v[k] = act_apply<ACT>(p.v[k]);
        }
        if (pre) st<V, NT>(pre, e, p);
        st<V, NT>(out, e, o);
    }
};

// delta *= act'(pre); from_delta = 1*from_delta + beta*delta; grad += alpha*delta.
// FIRST: this call is the first to write both targets in this backward pass, so they need not have
// been cleared: from_delta = beta*delta, grad = alpha*delta (what accumulating into zeros gives).
template<int ACT, bool FIRST = false>
struct ShortcutBackwardOp {
    float* delta;
    const float* pre;
    float* from_delta;
    float* grad;   // nullable
    float alpha, beta;
    template<int V> struct Regs { Pack<V> d, p, f, g; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.d = ld<V, NT>(delta, e);
        if constexpr (ACT != PXH_LINEAR) r.p = ld<V, NT>(pre, e);
        if constexpr (!FIRST) {
            r.f = ld<V, NT>(from_delta, e);
            if (grad) r.g = ld<V, NT>(grad, e);
        }
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const { finish_value<V, NT>(e, r); }
    // ... and returns what it left in grad (which must be there)
    template<int V, bool NT> __device__ Pack<V> finish_value(size_t e, const Regs<V>& r) const
    {
        Pack<V> d = r.d, f, g;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            if constexpr (ACT != PXH_LINEAR) d.v[k] = d.v[k] * act_grad<ACT>(r.p.v[k]);
            const float add = beta * d.v[k];
            const float ga = alpha * d.v[k];
            if constexpr (FIRST) {
                f.v[k] = add;
                g.v[k] = ga;
            } else {
                const float keep = 1.0f * r.f.v[k];
                f.v[k] = keep + add;
                if (grad) g.v[k] = r.g.v[k] + ga;
            }
        }
        if constexpr (ACT != PXH_LINEAR) st<V, NT>(delta, e, d);
        st<V, NT>(from_delta, e, f);
        if (grad) st<V, NT>(grad, e, g);
        return g;
    }
};

// The reference's index-mapped blend for operands of different shape.
__global__ __launch_bounds__(kBlock) void shortcut_mapped_kernel(uint32_t size, FastDiv by_w, FastDiv by_h, FastDiv by_c,
                                                                 int stride, int sample, int w1, int h1, int c1,
                                                                 const float* add, int w2, int h2, int c2, float s1,
                                                                 float s2, float* out)
{
    const uint32_t id = blockIdx.x * kBlock + threadIdx.x;
    if (id >= size) return;
    uint32_t rows, planes, i, j, k, b;
    by_w.divmod(id, rows, i);
    by_h.divmod(rows, planes, j);
    by_c.divmod(planes, b, k);
    const size_t oi = i * sample + static_cast<size_t>(w2) * (j * sample + static_cast<size_t>(h2) * (k + static_cast<size_t>(c2) * b));
    const size_t ai = i * stride + static_cast<size_t>(w1) * (j * stride + static_cast<size_t>(h1) * (k + static_cast<size_t>(c1) * b));
    const float po = s1 * out[oi];
    const float pa = s2 * add[ai];
    out[oi] = po + pa;
}

// ---------------------------------------------------------------- SGD with momentum
// The three BLAS calls of ConvLayer::update (include/ConvLayer.h:309-311, cuda 391-400) in one
// pass, one fp32 rounding per product and sum as there:
//   d += (-decay*batch) * w   (weights only);  w += (lr/batch) * d;  d *= momentum
struct SgdUpdateOp {
    float* w;
    float* d;
    float neg_decay_batch, rate, momentum;
    int apply_decay;
    template<int V> struct Regs { Pack<V> w, d; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.w = ld<V, NT>(w, e);
        r.d = ld<V, NT>(d, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> ow, od;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float g = r.d.v[k];
            if (apply_decay) {
                const float l2 = neg_decay_batch * r.w.v[k];
                g = g + l2;
            }
            const float step = rate * g;
            ow.v[k] = r.w.v[k] + step;
            od.v[k] = momentum * g;
        }
        st<V, NT>(w, e, ow);
        st<V, NT>(d, e, od);
    }
};

// ---------------------------------------------------------------- gradient rescale + clip
// Layer::backward's two helpers (include/Layer.h:385-397, 479-499; cuda/Layer.h:24-39):
//   norm = |x|_2;  if (norm > 0 && norm > threshold) x *= threshold / norm;  then clamp to +-clip.
// Pass 1: a fixed number of workgroups walk the tensor and leave one partial sum of squares each;
// pass 2: every workgroup adds up those partials (the same order everywhere), derives the factor
// and rewrites its part of the tensor; when nothing is to be done it leaves without touching it.
constexpr int kNormBlocks = 1024;     // 4 per compute unit; every workgroup of pass 2 re-adds this many partials
constexpr int kNormLoads = 8;         // 128-bit loads in flight per lane

// Per workgroup: the sum of squares and the largest magnitude (NaN-free; a NaN shows in the sum).
// (workgroup `block` of `blocks` that share the tensor; the result goes to *out)
//
// The 128-bit walk adds in an order that a flat kernel with one vector per lane can reproduce, so
// that a kernel which writes the tensor can leave these sums behind and spare the tensor a read:
//   group g    = the 256 values [256 g, 256 g + 256), one vector per lane of a wave; its sum is
//                q_g = wave_sum_by_rows over the lanes of ((x0^2 + x1^2) + x2^2) + x3^2
//                in fp32, values past the end counting as zero;
//   chain      = for workgroup b of B, vector u of kNormLoads, wave w:  T = sum over the steps i, in
//                order, of (double) q_g with g = ((i B + b) kNormLoads + u) 4 + w;
//   partial[b] = butterfly (offsets 16 .. 1) in fp64 over the workgroup's 32 chains, chain u*4 + w
//                in lane u*4 + w.
// norm_chains_kernel forms the same partials from stored group sums.
constexpr int kChains = kNormLoads * (kBlock / kWave);     // per workgroup
static_assert(kChains == 32, "the chains of a workgroup fill half a wave");

// The 32 chains of a workgroup, one per lane of the first half-wave (other lanes: anything), to the
// workgroup's partial; valid in lane 0.
__device__ __forceinline__ double chains_to_partial(double chain)
{
#pragma unroll
    for (int off = kChains / 2; off > 0; off >>= 1) chain += __shfl_xor(chain, off, kWave);
    return chain;
}

// What a walk over a tensor hands every vector it holds to, besides its own work: nothing, or the kernel
// that would read the tensor next (so that the tensor is read once for both).
struct NoSink {
    template<int V, bool NT> __device__ __forceinline__ void take(size_t, const Pack<V>&) const {}
};

template<int V, bool NT, typename Sink = NoSink>
__device__ __forceinline__ void sumsq_walk(const float* x, size_t n_vec, uint32_t block, uint32_t blocks, double2* out,
                                           const Sink& sink = Sink{})
{
    const size_t per_step = static_cast<size_t>(kBlock) * V * kNormLoads;
    if constexpr (V == 4) {
        __shared__ double chains[kChains];
        __shared__ float peaks[kBlock / kWave];
        double chain[kNormLoads];
#pragma unroll
        for (int u = 0; u < kNormLoads; ++u) chain[u] = 0.0;
        float peak = 0.0f;
        for (size_t base = static_cast<size_t>(block) * per_step; base < n_vec;
             base += static_cast<size_t>(blocks) * per_step) {
            Pack<V> v[kNormLoads];
            // a whole step has no branch between its loads (behind one each load is waited for before
            // the next goes out); only the last step of the tensor tests every vector
            if (base + per_step <= n_vec) {
#pragma unroll
                for (int u = 0; u < kNormLoads; ++u)
                    v[u] = ld<V, NT>(x, base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V);
            } else {
#pragma unroll
                for (int u = 0; u < kNormLoads; ++u) {
                    const size_t e = base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V;
#pragma unroll
                    for (int k = 0; k < V; ++k) v[u].v[k] = 0.0f;
                    if (e < n_vec) v[u] = ld<V, NT>(x, e);
                }
            }
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u) {
                peak = fmaxf(peak, peak_of(v[u]));
                chain[u] += static_cast<double>(wave_sum_by_rows(square_sum(v[u])));
            }
            if constexpr (!std::is_same_v<Sink, NoSink>) {
#pragma unroll
                for (int u = 0; u < kNormLoads; ++u) {
                    const size_t e = base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V;
                    if (e < n_vec) sink.template take<V, NT>(e, v[u]);
                }
            }
        }
        peak = wave_max(peak);
        const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
        if (lane == 0) {
            peaks[wave] = peak;
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u) chains[u * (kBlock / kWave) + wave] = chain[u];
        }
        __syncthreads();
        if (wave == 0) {
            const double total = chains_to_partial(chains[lane & (kChains - 1)]);
            if (lane == 0) {
                float top = peaks[0];
#pragma unroll
                for (int w = 1; w < kBlock / kWave; ++w) top = fmaxf(top, peaks[w]);
                *out = make_double2(total, static_cast<double>(top));
            }
        }
    } else {
        // one value per lane (a tensor that is not 16-byte aligned or not a multiple of 4 long):
        // fp32 over a step, fp64 over the steps and the workgroup
        __shared__ double slots[kBlock / kWave];
        __shared__ float peaks[kBlock / kWave];
        double s = 0.0;
        float peak = 0.0f;
        for (size_t base = static_cast<size_t>(block) * per_step; base < n_vec;
             base += static_cast<size_t>(blocks) * per_step) {
            float a = 0.0f;
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u) {
                const size_t e = base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V;
                if (e < n_vec) {
                    const Pack<V> v = ld<V, NT>(x, e);
#pragma unroll
                    for (int k = 0; k < V; ++k) {
                        a += v.v[k] * v.v[k];
                        peak = fmaxf(peak, fabsf(v.v[k]));
                    }
                }
            }
            s += static_cast<double>(a);
        }
        peak = wave_max(peak);
        if ((threadIdx.x & (kWave - 1)) == 0) peaks[threadIdx.x / kWave] = peak;
        const double total = block_sum(s, slots);       // synchronises the workgroup twice
        if (threadIdx.x == 0) {
            float top = peaks[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) top = fmaxf(top, peaks[w]);
            *out = make_double2(total, static_cast<double>(top));
        }
    }
}

// Group sums that a kernel left while writing the tensor (float2: sum of squares, largest
// magnitude), to the partials of the walk above: one lane per chain.
__global__ __launch_bounds__(kBlock) void norm_chains_kernel(const float2* groups, size_t n_groups, uint32_t blocks,
                                                            double2* partial)
{
    const uint32_t chain = blockIdx.x * kBlock + threadIdx.x;      // = b * kChains + u * 4 + w
    const size_t per_step = static_cast<size_t>(blocks) * kChains;
    double total = 0.0;
    float peak = 0.0f;
    if (chain < per_step) {
        for (size_t g = chain; g < n_groups; g += per_step) {
            const float2 q = groups[g];
            total += static_cast<double>(q.x);
            peak = fmaxf(peak, q.y);
        }
    }
    total = chains_to_partial(total);
#pragma unroll
    for (int off = kChains / 2; off > 0; off >>= 1) peak = fmaxf(peak, __shfl_xor(peak, off, kWave));
    if ((threadIdx.x & (kChains - 1)) == 0 && chain < per_step)
        partial[chain / kChains] = make_double2(total, static_cast<double>(peak));
}

template<int V, bool NT>
__global__ __launch_bounds__(kBlock) void sumsq_partial_kernel(const float* x, size_t n_vec, double2* partial)
{
    sumsq_walk<V, NT>(x, n_vec, blockIdx.x, gridDim.x, partial + blockIdx.x);
}

// The plan of the rewrite (plan_from_totals), formed by every workgroup for itself from the same
// partials in the same order, so all arrive at the same one.
__device__ __forceinline__ RescalePlan rescale_plan(const double2* partial, int partials, float threshold, float clip)
{
    __shared__ double sums[kBlock / kWave];
    __shared__ double tops[kBlock / kWave];
    double s = 0.0, top = 0.0;
    for (int j = threadIdx.x; j < partials; j += kBlock) {
        const double2 p = partial[j];
        s += p.x;
        top = fmax(top, p.y);
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        s += __shfl_xor(s, off, kWave);
        top = fmax(top, __shfl_xor(top, off, kWave));
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        sums[threadIdx.x / kWave] = s;
        tops[threadIdx.x / kWave] = top;
    }
    __syncthreads();
    double total = 0.0;
    float peak = 0.0f;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        total += sums[w];
        peak = fmaxf(peak, static_cast<float>(tops[w]));
    }
    return plan_from_totals(total, peak, threshold, clip);
}

// x = clamp(factor * x); leaves without touching the tensor when there is nothing to do.  The grid
// is the reduction's capped one and strides over the tensor.
template<int V, bool NT, typename Sink = NoSink>
__device__ __forceinline__ void rescale_walk(float* x, size_t n_vec, const double2* partial, int partials,
                                             uint32_t block, uint32_t blocks, float threshold, float clip,
                                             float* norm_out, const Sink& sink = Sink{})
{
    const RescalePlan plan = rescale_plan(partial, partials, threshold, clip);
    if (norm_out && block == 0 && threadIdx.x == 0) *norm_out = plan.norm;
    if (!plan.work) return;
    const float factor = plan.factor;
    const size_t per_step = static_cast<size_t>(kBlock) * V * kNormLoads;
    for (size_t base = static_cast<size_t>(block) * per_step; base < n_vec;
         base += static_cast<size_t>(blocks) * per_step) {
        Pack<V> v[kNormLoads];
        const auto rewrite = [&](Pack<V>& p) {
#pragma unroll
            for (int k = 0; k < V; ++k) p.v[k] = rescaled_clipped(p.v[k], factor, clip);
        };
        if (base + per_step <= n_vec) {      // a whole step: no branch between its loads
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u)
                v[u] = ld<V, NT>(x, base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V);
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u) {
                rewrite(v[u]);
                st<V, NT>(x, base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V, v[u]);
                sink.template take<V, NT>(base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V, v[u]);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kNormLoads; ++u) {
                const size_t e = base + (static_cast<size_t>(u) * kBlock + threadIdx.x) * V;
                if (e < n_vec) {
                    v[u] = ld<V, NT>(x, e);
                    rewrite(v[u]);
                    st<V, NT>(x, e, v[u]);
                    sink.template take<V, NT>(e, v[u]);
                }
            }
        }
    }
}

template<int V, bool NT>
__global__ __launch_bounds__(kBlock) void rescale_clip_kernel(float* x, size_t n_vec, const double2* partial,
                                                              int partials, float threshold, float clip,
                                                              float* norm_out)
{
    rescale_walk<V, NT>(x, n_vec, partial, partials, blockIdx.x, gridDim.x, threshold, clip, norm_out);
}

// ---- Layer::backward's rescale + clip of a shortcut's delta with the shortcut's backward in the same passes ----
// A shortcut that is the first to write its two targets in the backward pass (ShortcutBackwardOp<LINEAR, true>)
// leaves in them plain functions of its delta.  The pass that adds up the delta's norm therefore also writes
// them, as if nothing had to change; the second launch forms the plan, leaves at once when that was right, and
// otherwise rewrites the delta and both targets from it: the values of pxh_rescale_clip followed by
// pxh_shortcut_backward_first either way, with the delta read once where it had been read twice.
struct ShortcutFirstSink {
    float* from_delta;
    float* grad;   // nullable
    float alpha, beta;
    template<int V, bool NT> __device__ __forceinline__ void take(size_t e, const Pack<V>& d) const
    {
        Pack<V> f, g;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            f.v[k] = beta * d.v[k];
            g.v[k] = alpha * d.v[k];
        }
        st<V, NT>(from_delta, e, f);
        if (grad) st<V, NT>(grad, e, g);
    }
};

template<bool NT, typename Sink>
__global__ __launch_bounds__(kBlock) void sumsq_sink_kernel(const float* x, size_t n_vec, double2* partial, Sink sink)
{
    sumsq_walk<4, NT, Sink>(x, n_vec, blockIdx.x, gridDim.x, partial + blockIdx.x, sink);
}

template<bool NT, typename Sink>
__global__ __launch_bounds__(kBlock) void rescale_clip_sink_kernel(float* x, size_t n_vec, const double2* partial,
                                                                   int partials, float threshold, float clip,
                                                                   float* norm_out, Sink sink)
{
    rescale_walk<4, NT, Sink>(x, n_vec, partial, partials, blockIdx.x, gridDim.x, threshold, clip, norm_out, sink);
}

// The same two passes over up to kRescaleTensors tensors per launch (the update hooks of a model run
// on every layer's update buffers, three per convolution).  Every tensor gets the workgroups, the
// walk and therefore the sums of its single call: the results are the same bit for bit.
constexpr int kRescaleTensors = 32;

struct RescaleTable {
    float* x[kRescaleTensors];
    unsigned long long n[kRescaleTensors];
    uint32_t first_block[kRescaleTensors + 1];     // also the tensor's first partial
    uint32_t vector_mask;                          // bit i: 16-byte aligned and a multiple of 4 long
    uint32_t past_cache_mask;
    int count;
    float* norms;                                  // nullable: norms[first_tensor + i]
    int first_tensor;
};

__device__ __forceinline__ int tensor_of_block(const uint32_t* first_block, int count, uint32_t block)
{
    int lo = 0, hi = count - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (first_block[mid] <= block) lo = mid; else hi = mid - 1;
    }
    return lo;
}

__global__ __launch_bounds__(kBlock) void multi_sumsq_kernel(RescaleTable t, double2* partial)
{
    const int i = tensor_of_block(t.first_block, t.count, blockIdx.x);
    const uint32_t block = blockIdx.x - t.first_block[i], blocks = t.first_block[i + 1] - t.first_block[i];
    double2* out = partial + blockIdx.x;
    if (!((t.vector_mask >> i) & 1u)) sumsq_walk<1, false>(t.x[i], t.n[i], block, blocks, out);
    else if ((t.past_cache_mask >> i) & 1u) sumsq_walk<4, true>(t.x[i], t.n[i], block, blocks, out);
    else sumsq_walk<4, false>(t.x[i], t.n[i], block, blocks, out);
}

__global__ __launch_bounds__(kBlock) void multi_rescale_kernel(RescaleTable t, const double2* partial, float threshold,
                                                               float clip)
{
    const int i = tensor_of_block(t.first_block, t.count, blockIdx.x);
    const uint32_t block = blockIdx.x - t.first_block[i], blocks = t.first_block[i + 1] - t.first_block[i];
    const double2* mine = partial + t.first_block[i];
    float* norm_out = t.norms ? t.norms + t.first_tensor + i : nullptr;
    if (!((t.vector_mask >> i) & 1u))
        rescale_walk<1, false>(t.x[i], t.n[i], mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
    else if ((t.past_cache_mask >> i) & 1u)
        rescale_walk<4, true>(t.x[i], t.n[i], mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
    else
        rescale_walk<4, false>(t.x[i], t.n[i], mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
}

// ---------------------------------------------------------------- Adam
// One fp32 rounding per BLAS call of the reference sequence (include/cuda/Adam.h:49-90).
struct AdamUpdateOp {
    float* w;
    float* d;
    float* m;
    float* v;
    float inv_batch, neg_decay, beta1, beta2, a1, a2, c1, c2, lr, eps;
    float neg_lr_decay;     // -(lr * decay), for the decoupled form only
    int apply_decay;        // 0: none; 1: folded into the update before the moments (the reference); 2: decoupled
    template<int V> struct Regs { Pack<V> w, d, m, v; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.w = ld<V, NT>(w, e);
        r.d = ld<V, NT>(d, e);
        r.m = ld<V, NT>(m, e);
        r.v = ld<V, NT>(v, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> ow, om, ov, od;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float g = r.d.v[k] * inv_batch;
            if (apply_decay == 1) {
                const float l2 = neg_decay * r.w.v[k];
                g = g + l2;
            }
            float mi = r.m.v[k] * beta1;
            float vi = r.v.v[k] * beta2;
            const float am = a1 * g;
            mi = mi + am;
            const float g2 = g * g;
            const float av = a2 * g2;
            vi = vi + av;
            const float mhat = mi / c1;
            const float vhat = vi / c2;
            const float step = lr * mhat / (sqrtf(vhat) + eps);
            float wi = r.w.v[k] + step;
            if (apply_decay == 2) {
                // decoupled: the weight shrinks by lr * decay of its old value, outside the moments
                const float shrink = neg_lr_decay * r.w.v[k];
                wi = wi + shrink;
            }
            ow.v[k] = wi;
            om.v[k] = mi;
            ov.v[k] = vi;
            od.v[k] = 0.0f;
        }
        st<V, NT>(w, e, ow);
        st<V, NT>(m, e, om);
        st<V, NT>(v, e, ov);
        st<V, NT>(d, e, od);
    }
};

// ---------------------------------------------------------------- many parameter tensors, few launches
// The engine keeps every layer's weights, biases and scales in buffers of their own and updates them
// one by one (include/cuda/ConvLayer.h:370-413): 222 tensors for YOLOv3, two thirds of them smaller
// than one workgroup's worth.  A launch here takes up to kMultiTensors of them: the table travels by
// value, workgroup b finds its tensor by bisection over the first workgroup of each, and runs the
// same per-element operation on 1024 elements of it.
constexpr int kMultiTensors = 32;
constexpr uint32_t kMultiPerBlock = kBlock * 4;

struct MultiTable {
    float* stream[4][kMultiTensors];               // the tensor's buffers, in the operation's own order
    unsigned long long n[kMultiTensors];
    uint32_t first_block[kMultiTensors + 1];
    uint32_t decay_mask;                           // bit i: tensor i takes the weight decay
    uint32_t past_cache_mask;                      // bit i: tensor i is too large to stay cached
    uint32_t vector_mask;                          // bit i: all buffers of tensor i are 16-byte aligned
    int count;
};

struct AdamMaker {
    AdamUpdateOp base;
    __device__ AdamUpdateOp operator()(const MultiTable& t, int i) const
    {
        AdamUpdateOp op = base;
        op.w = t.stream[0][i]; op.d = t.stream[1][i]; op.m = t.stream[2][i]; op.v = t.stream[3][i];
        op.apply_decay = (t.decay_mask >> i) & 1u;
        return op;
    }
};

struct SgdMaker {
    SgdUpdateOp base;
    __device__ SgdUpdateOp operator()(const MultiTable& t, int i) const
    {
        SgdUpdateOp op = base;
        op.w = t.stream[0][i]; op.d = t.stream[1][i];
        op.apply_decay = (t.decay_mask >> i) & 1u;
        return op;
    }
};

struct FillMaker {
    float value;
    __device__ FillOp operator()(const MultiTable& t, int i) const { return FillOp{ t.stream[0][i], value }; }
};

template<typename Maker>
__global__ __launch_bounds__(kBlock) void multi_tensor_kernel(MultiTable t, Maker make)
{
    const int lo = tensor_of_block(t.first_block, t.count, blockIdx.x);
    const auto op = make(t, lo);
    const size_t n = t.n[lo];
    const size_t e = (static_cast<size_t>(blockIdx.x - t.first_block[lo]) * kBlock + threadIdx.x) * 4;
    if (e >= n) return;
    using Op = decltype(make(t, 0));
    if (((t.vector_mask >> lo) & 1u) && e + 4 <= n) {
        typename Op::template Regs<4> r;
        if ((t.past_cache_mask >> lo) & 1u) {
            op.template load<4, true>(e, r);
            op.template finish<4, true>(e, r);
        } else {
            op.template load<4, false>(e, r);
            op.template finish<4, false>(e, r);
        }
    } else {
        for (size_t k = e; k < n && k < e + 4; ++k) {
            typename Op::template Regs<1> r;
            op.template load<1, false>(k, r);
            op.template finish<1, false>(k, r);
        }
    }
}

// Runs `make`'s operation over `count` tensors (host arrays of device pointers and sizes).
template<int STREAMS, typename Maker>
int launch_multi(const char* who, int count, float* const* const* buffers, const size_t* n, const int* apply_decay,
                 int bytes_per_elem, const Maker& make, hipStream_t stream, size_t streaming_from = kStreamingBytes)
{
    for (int begin = 0; begin < count; begin += kMultiTensors) {
        MultiTable t{};
        const int part = count - begin < kMultiTensors ? count - begin : kMultiTensors;
        unsigned long long blocks = 0;
        int used = 0;
        for (int i = 0; i < part; ++i) {
            const size_t len = n[begin + i];
            if (len == 0) continue;
            bool aligned = true;
            for (int k = 0; k < STREAMS; ++k) {
                float* ptr = buffers[k][begin + i];
                if (!ptr) return fail_invalid("%s: null pointer for tensor %d", who, begin + i);
                aligned = aligned && aligned16(ptr);
                t.stream[k][used] = ptr;
            }
            t.n[used] = len;
            t.first_block[used] = static_cast<uint32_t>(blocks);
            if (apply_decay && apply_decay[begin + i]) t.decay_mask |= 1u << used;
            if (len * static_cast<size_t>(bytes_per_elem) >= streaming_from) t.past_cache_mask |= 1u << used;
            if (aligned) t.vector_mask |= 1u << used;
            blocks += (len + kMultiPerBlock - 1) / kMultiPerBlock;
            ++used;
        }
        if (used == 0) continue;
        if (blocks > 0x7fffffffull) {
            set_error("%s: more than 2^31 workgroups in one launch", who);
            return PXH_ERR_UNSUPPORTED;
        }
        t.first_block[used] = static_cast<uint32_t>(blocks);
        t.count = used;
        hipLaunchKernelGGL((multi_tensor_kernel<Maker>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, t,
                           make);
        const int rc = check_launch(who);
        if (rc) return rc;
    }
    return PXH_OK;
}

// ---------------------------------------------------------------- the same over a table kept on the device
// A by-value table holds 32 tensors, so a model's 222 parameter tensors still take 7 launches per
// operation.  A table built once and kept in device memory (pxh_tensor_table_create) takes them all in
// ONE: the launch carries only its address.  Workgroup b copies the list of first workgroups into LDS
// (one coalesced load), finds its tensor there by bisection and fetches that tensor's record; the
// per-element work and the order of every sum are those of the single call.
constexpr int kMaxTableTensors = 2048;

struct __attribute__((aligned(16))) TensorRecord {     // 64 bytes
    float* stream[4];               // the tensor's buffers, in the operation's own order
    unsigned long long n;
    uint32_t decay;                 // the weight decay applies
    uint32_t vector;                // every buffer is 16-byte aligned: the 128-bit form
    uint32_t norm_vector;           // stream[0] is 16-byte aligned and n % 4 == 0: the 128-bit form of the norm
    uint32_t pad[3];
};

struct TableView {
    const TensorRecord* records;
    const uint32_t* first_block;        // [count + 1] workgroups of the streaming operations
    const uint32_t* first_norm_block;   // [count + 1] workgroups of the norm and rescale passes, = first partials
    double2* partial;                   // sums of squares and peaks, one per workgroup of the norm pass
    int count;
};

// The tensor workgroup `block` works on; `firsts` is LDS for count + 1 entries.
__device__ __forceinline__ int table_tensor_of_block(const uint32_t* first_block, int count, uint32_t block, uint32_t* firsts)
{
    for (int i = threadIdx.x; i <= count; i += kBlock) firsts[i] = first_block[i];
    __syncthreads();
    return tensor_of_block(firsts, count, block);
}

struct AdamFromRecord {
    AdamUpdateOp base;
    __device__ AdamUpdateOp operator()(const TensorRecord& r) const
    {
        AdamUpdateOp op = base;
        op.w = r.stream[0]; op.d = r.stream[1]; op.m = r.stream[2]; op.v = r.stream[3];
        op.apply_decay = static_cast<int>(r.decay);
        return op;
    }
};

struct SgdFromRecord {
    SgdUpdateOp base;
    __device__ SgdUpdateOp operator()(const TensorRecord& r) const
    {
        SgdUpdateOp op = base;
        op.w = r.stream[0]; op.d = r.stream[1];
        op.apply_decay = static_cast<int>(r.decay);
        return op;
    }
};

struct FillFromRecord {
    float value;
    __device__ FillOp operator()(const TensorRecord& r) const { return FillOp{ r.stream[0], value }; }
};

// `streaming_elems`: tensors of at least this many elements go past the caches (0: all of them).
// A workgroup takes kTableChunks consecutive 1024-element chunks of its tensor, so that the cost of
// finding the tensor is spread over four times the elements (it is what the single call does not pay).
constexpr int kTableChunks = 4;
constexpr uint32_t kTablePerBlock = kMultiPerBlock * kTableChunks;

template<typename Maker>
__global__ __launch_bounds__(kBlock) void table_stream_kernel(TableView t, Maker make, unsigned long long streaming_elems)
{
    __shared__ uint32_t firsts[kMaxTableTensors + 1];
    const int i = table_tensor_of_block(t.first_block, t.count, blockIdx.x, firsts);
    const TensorRecord r = t.records[i];
    const auto op = make(r);
    const size_t n = r.n;
    using Op = decltype(make(r));
    const size_t base = static_cast<size_t>(blockIdx.x - firsts[i]) * kTablePerBlock + static_cast<size_t>(threadIdx.x) * 4;
    if (r.vector && base + (kTableChunks - 1) * kMultiPerBlock + 4 <= n) {
        // every chunk holds a whole vector for this lane: the loads of all of them go out together
        typename Op::template Regs<4> regs[kTableChunks];
        if (n >= streaming_elems) {
#pragma unroll
            for (int c = 0; c < kTableChunks; ++c) op.template load<4, true>(base + c * kMultiPerBlock, regs[c]);
#pragma unroll
            for (int c = 0; c < kTableChunks; ++c) op.template finish<4, true>(base + c * kMultiPerBlock, regs[c]);
        } else {
#pragma unroll
            for (int c = 0; c < kTableChunks; ++c) op.template load<4, false>(base + c * kMultiPerBlock, regs[c]);
#pragma unroll
            for (int c = 0; c < kTableChunks; ++c) op.template finish<4, false>(base + c * kMultiPerBlock, regs[c]);
        }
        return;
    }
    for (int c = 0; c < kTableChunks; ++c) {
        const size_t e = base + c * kMultiPerBlock;
        if (e >= n) return;
        if (r.vector && e + 4 <= n) {
            typename Op::template Regs<4> regs;
            op.template load<4, false>(e, regs);
            op.template finish<4, false>(e, regs);
        } else {
            for (size_t k = e; k < n && k < e + 4; ++k) {
                typename Op::template Regs<1> regs;
                op.template load<1, false>(k, regs);
                op.template finish<1, false>(k, regs);
            }
        }
    }
}

__global__ __launch_bounds__(kBlock) void table_sumsq_kernel(TableView t)
{
    __shared__ uint32_t firsts[kMaxTableTensors + 1];
    const int i = table_tensor_of_block(t.first_norm_block, t.count, blockIdx.x, firsts);
    const TensorRecord r = t.records[i];
    const uint32_t block = blockIdx.x - firsts[i], blocks = firsts[i + 1] - firsts[i];
    double2* out = t.partial + blockIdx.x;
    if (!r.norm_vector) sumsq_walk<1, false>(r.stream[0], r.n, block, blocks, out);
    else if (r.n * 4 >= kStreamingBytes) sumsq_walk<4, true>(r.stream[0], r.n, block, blocks, out);
    else sumsq_walk<4, false>(r.stream[0], r.n, block, blocks, out);
}

__global__ __launch_bounds__(kBlock) void table_rescale_kernel(TableView t, float threshold, float clip, float* norms)
{
    __shared__ uint32_t firsts[kMaxTableTensors + 1];
    const int i = table_tensor_of_block(t.first_norm_block, t.count, blockIdx.x, firsts);
    const TensorRecord r = t.records[i];
    const uint32_t block = blockIdx.x - firsts[i], blocks = firsts[i + 1] - firsts[i];
    const double2* mine = t.partial + firsts[i];
    float* norm_out = norms ? norms + i : nullptr;
    if (!r.norm_vector)
        rescale_walk<1, false>(r.stream[0], r.n, mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
    else if (r.n * 4 >= kStreamingBytes)
        rescale_walk<4, true>(r.stream[0], r.n, mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
    else
        rescale_walk<4, false>(r.stream[0], r.n, mine, static_cast<int>(blocks), block, blocks, threshold, clip, norm_out);
}

struct AdamStepOp {
    float* x;
    const float* m;
    const float* v;
    float c1, c2, rate, eps;
    template<int V> struct Regs { Pack<V> x, m, v; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
        r.x = ld<V, NT>(x, e);
        r.m = ld<V, NT>(m, e);
        r.v = ld<V, NT>(v, e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> o;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const float mhat = r.m.v[k] / c1;
            const float vhat = r.v.v[k] / c2;
            const float step = rate * mhat / (sqrtf(vhat) + eps);
            o.v[k] = r.x.v[k] + step;
        }
        st<V, NT>(x, e, o);
    }
};

// ---------------------------------------------------------------- a mix of streams, nothing else
// R streams read, their sum written to W streams: the cost of a read/write mix itself (test hook).
template<int R, int W>
struct MixOp {
    const float* in[4];
    float* out[4];
    template<int V> struct Regs { Pack<V> x[R]; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const
    {
#pragma unroll
        for (int i = 0; i < R; ++i) r.x[i] = ld<V, NT>(in[i], e);
    }
    template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>& r) const
    {
        Pack<V> sum = r.x[0];
#pragma unroll
        for (int i = 1; i < R; ++i) {
#pragma unroll
            for (int k = 0; k < V; ++k) sum.v[k] += r.x[i].v[k];
        }
#pragma unroll
        for (int i = 0; i < W; ++i) st<V, NT>(out[i], e, sum);
    }
};

template<int R, int W>
int launch_mix(size_t n, const float* const* in, float* const* out, hipStream_t s)
{
    MixOp<R, W> op{};
    for (int i = 0; i < R; ++i) op.in[i] = in[i];
    for (int i = 0; i < W; ++i) op.out[i] = out[i];
    // launched as the library launches an operation of that many streams (two vectors per lane for 4 + 4)
    return launch_stream("pxh_debug_stream_mix", n, true, 4 * (R + W), op, s, kStreamingBytes, R + W >= 8);
}

}  // namespace
}  // namespace pxh

using namespace pxh;

namespace pxh {
namespace {
// The tensor as it is: what a kernel of this file that cannot leave group sums itself is followed by.
struct GroupsOnlyOp {
    const float* x;
    template<int V> struct Regs { Pack<V> x; };
    template<int V, bool NT> __device__ void load(size_t e, Regs<V>& r) const { r.x = ld<V, NT>(x, e); }
    template<int V, bool NT> __device__ void finish(size_t, const Regs<V>&) const {}
    template<int V, bool NT> __device__ Pack<V> finish_value(size_t, const Regs<V>& r) const { return r.x; }
};

// The norm pass reads a tensor 128 bits at a time under this condition, and only then do group sums
// describe it; otherwise nothing is written to, or read from, a group buffer.
inline bool has_groups(const float* x, size_t n) { return aligned16(x) && n % 4 == 0; }

}  // namespace
}  // namespace pxh

extern "C" {

int pxh_activate(int activation, float* x, size_t n, void* stream)
{
    if (!x && n) return fail_invalid("pxh_activate: null pointer");
    int rc = PXH_OK;
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if constexpr (ACT == PXH_LINEAR) return;
        rc = launch_stream("pxh_activate", n, aligned16(x), 8, ActivateOp<ACT>{ x }, as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_activate: unknown activation %d", activation);
    return rc;
}

int pxh_gradient(int activation, const float* x, size_t n, float* delta, void* stream)
{
    if ((!x || !delta) && n) return fail_invalid("pxh_gradient: null pointer");
    int rc = PXH_OK;
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if constexpr (ACT == PXH_LINEAR) return;
        rc = launch_stream("pxh_gradient", n, aligned16(x) && aligned16(delta), 12, GradientOp<ACT>{ x, delta },
                           as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_gradient: unknown activation %d", activation);
    return rc;
}

int pxh_fill_f32(float* x, size_t n, float value, void* stream)
{
    if (!x && n) return fail_invalid("pxh_fill_f32: null pointer");
    return launch_stream("pxh_fill_f32", n, aligned16(x), 4, FillOp{ x, value }, as_stream(stream), kFillStreamingBytes);
}

int pxh_fill_i32(int* x, size_t n, int value, void* stream)
{
    if (!x && n) return fail_invalid("pxh_fill_i32: null pointer");
    float bits;
    static_assert(sizeof(bits) == sizeof(value), "int and float must have the same size");
    __builtin_memcpy(&bits, &value, sizeof(bits));
    return launch_stream("pxh_fill_i32", n, aligned16(x), 4, FillOp{ reinterpret_cast<float*>(x), bits },
                         as_stream(stream), kFillStreamingBytes);
}

int pxh_constrain(int n, float alpha, float* x, void* stream)
{
    if (n < 0 || (!x && n)) return fail_invalid("pxh_constrain: bad argument");
    return launch_stream("pxh_constrain", static_cast<size_t>(n), aligned16(x), 8, ConstrainOp{ x, alpha },
                         as_stream(stream));
}

int pxh_mul(int n, const float* x, float* y, void* stream)
{
    if (n < 0 || ((!x || !y) && n)) return fail_invalid("pxh_mul: bad argument");
    return launch_stream("pxh_mul", static_cast<size_t>(n), aligned16(x) && aligned16(y), 12, MulOp{ x, y },
                         as_stream(stream));
}

int pxh_axpy(size_t n, float alpha, const float* x, float* y, void* stream)
{
    if ((!x || !y) && n) return fail_invalid("pxh_axpy: null pointer");
    return launch_stream("pxh_axpy", n, aligned16(x) && aligned16(y), 12, AxpyOp{ x, y, alpha }, as_stream(stream));
}

int pxh_route_forward(const float* layer_output, float* route_output, int batch, int layer_outputs,
                      int route_outputs, int offset, void* stream)
{
    int rc = check_route("pxh_route_forward", layer_output, route_output, batch, layer_outputs, route_outputs, offset);
    if (rc) return rc;
    const size_t n = static_cast<size_t>(batch) * layer_outputs;
    if (n == 0) return PXH_OK;
    const bool vec = aligned16(layer_output) && aligned16(route_output) && layer_outputs % 4 == 0 &&
                     route_outputs % 4 == 0 && offset % 4 == 0;
    return launch_stream("pxh_route_forward", n, vec, 8,
                         RouteOp<false>{ layer_output, route_output, FastDiv(layer_outputs),
                                         static_cast<uint32_t>(route_outputs), static_cast<uint32_t>(offset) },
                         as_stream(stream));
}

int pxh_route_backward(const float* route_delta, float* layer_delta, int batch, int layer_outputs,
                       int route_outputs, int offset, void* stream)
{
    int rc = check_route("pxh_route_backward", route_delta, layer_delta, batch, layer_outputs, route_outputs, offset);
    if (rc) return rc;
    const size_t n = static_cast<size_t>(batch) * layer_outputs;
    if (n == 0) return PXH_OK;
    const bool vec = aligned16(route_delta) && aligned16(layer_delta) && layer_outputs % 4 == 0 &&
                     route_outputs % 4 == 0 && offset % 4 == 0;
    return launch_stream("pxh_route_backward", n, vec, 12,
                         RouteOp<true>{ route_delta, layer_delta, FastDiv(layer_outputs),
                                        static_cast<uint32_t>(route_outputs), static_cast<uint32_t>(offset) },
                         as_stream(stream));
}

int pxh_shortcut(int batch, int w1, int h1, int c1, const float* add, int w2, int h2, int c2, float s1, float s2,
                 float* out, void* stream)
{
    if (!add || !out) return fail_invalid("pxh_shortcut: null pointer");
    if (batch <= 0 || w1 <= 0 || h1 <= 0 || c1 <= 0 || w2 <= 0 || h2 <= 0 || c2 <= 0)
        return fail_invalid("pxh_shortcut: dimensions must be positive");
    int stride = w1 / w2; if (stride < 1) stride = 1;
    int sample = w2 / w1; if (sample < 1) sample = 1;
    // the CPU layer rejects these (PX_CHECK in ShortcutLayer::shortcut)
    if (stride != h1 / h2) return fail_invalid("pxh_shortcut: stride must be equal in x and y direction");
    if (sample != h2 / h1) return fail_invalid("pxh_shortcut: sample must be equal in x and y direction");
    const int minw = w1 < w2 ? w1 : w2, minh = h1 < h2 ? h1 : h2, minc = c1 < c2 ? c1 : c2;
    const unsigned long long size = 1ull * batch * minw * minh * minc;
    if (size >= (1ull << 31)) {
        set_error("pxh_shortcut: too many elements");
        return PXH_ERR_UNSUPPORTED;
    }
    if (w1 == w2 && h1 == h2 && c1 == c2) {
        // same shape: identity index maps, out = s1*out + s2*add as a flat stream
        return launch_stream("pxh_shortcut", static_cast<size_t>(size), aligned16(add) && aligned16(out), 12,
                             ShortcutForwardOp<PXH_LINEAR>{ out, add, out, nullptr, s1, s2 }, as_stream(stream));
    }
    hipLaunchKernelGGL(shortcut_mapped_kernel, dim3(grid_for(size, kBlock)), dim3(kBlock), 0, as_stream(stream),
                       static_cast<uint32_t>(size), FastDiv(minw), FastDiv(minh), FastDiv(minc), stride, sample, w1,
                       h1, c1, add, w2, h2, c2, s1, s2, out);
    return check_launch("pxh_shortcut");
}

int pxh_shortcut_forward(const float* input, const float* from_output, float* output, float* pre_activation,
                         size_t n, float alpha, float beta, int activation, void* stream)
{
    if ((!input || !from_output || !output) && n) return fail_invalid("pxh_shortcut_forward: null pointer");
    int rc = PXH_OK;
    const bool vec = aligned16(input) && aligned16(from_output) && aligned16(output) && aligned16(pre_activation);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        rc = launch_stream("pxh_shortcut_forward", n, vec, pre_activation ? 16 : 12,
                           ShortcutForwardOp<ACT>{ input, from_output, output, pre_activation, alpha, beta },
                           as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_shortcut_forward: unknown activation %d", activation);
    return rc;
}

int pxh_shortcut_backward(float* delta, const float* pre_activation, float* from_delta, float* grad, size_t n,
                          float alpha, float beta, int activation, void* stream)
{
    if ((!delta || !from_delta) && n) return fail_invalid("pxh_shortcut_backward: null pointer");
    if (activation != PXH_LINEAR && !pre_activation && n)
        return fail_invalid("pxh_shortcut_backward: pre_activation is required for a non-linear activation");
    int rc = PXH_OK;
    const bool vec = aligned16(delta) && aligned16(pre_activation) && aligned16(from_delta) && aligned16(grad);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        rc = launch_stream("pxh_shortcut_backward", n, vec, grad ? 20 : 12,
                           ShortcutBackwardOp<ACT>{ delta, pre_activation, from_delta, grad, alpha, beta },
                           as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_shortcut_backward: unknown activation %d", activation);
    return rc;
}

int pxh_shortcut_backward_first(float* delta, const float* pre_activation, float* from_delta, float* grad, size_t n,
                                float alpha, float beta, int activation, void* stream)
{
    if ((!delta || !from_delta) && n) return fail_invalid("pxh_shortcut_backward_first: null pointer");
    if (activation != PXH_LINEAR && !pre_activation && n)
        return fail_invalid("pxh_shortcut_backward_first: pre_activation is required for a non-linear activation");
    if (from_delta == grad && n)
        return fail_invalid("pxh_shortcut_backward_first: from_delta and grad must be distinct when both are overwritten");
    int rc = PXH_OK;
    const bool vec = aligned16(delta) && aligned16(pre_activation) && aligned16(from_delta) && aligned16(grad);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        rc = launch_stream("pxh_shortcut_backward_first", n, vec, grad ? 12 : 8,
                           ShortcutBackwardOp<ACT, true>{ delta, pre_activation, from_delta, grad, alpha, beta },
                           as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_shortcut_backward_first: unknown activation %d", activation);
    return rc;
}

int pxh_sgd_update(size_t n, float* w, float* d, int batch, float lr, float momentum, float decay, int apply_decay,
                   void* stream)
{
    if (batch <= 0) return fail_invalid("pxh_sgd_update: batch must be positive");
    if ((!w || !d) && n) return fail_invalid("pxh_sgd_update: null pointer");
    const SgdUpdateOp op{ w, d, -decay * static_cast<float>(batch), lr / static_cast<float>(batch), momentum,
                          apply_decay };
    return launch_stream("pxh_sgd_update", n, aligned16(w) && aligned16(d), 16, op, as_stream(stream));
}

// ---------------------------------------------------------------- norm + peak from the writing kernel
size_t pxh_norm_groups_bytes(size_t n)
{
    return (n + kGroupValues - 1) / kGroupValues * sizeof(float2);
}

int pxh_norm_groups(const float* x, size_t n, void* groups, void* stream)
{
    if ((!x || !groups) && n) return fail_invalid("pxh_norm_groups: null pointer");
    if (!has_groups(x, n)) return PXH_OK;
    return launch_stream_groups("pxh_norm_groups", n, 4, GroupsOnlyOp{ x }, static_cast<float2*>(groups),
                                as_stream(stream));
}

int pxh_axpy_norm(size_t n, float alpha, const float* x, float* y, void* y_groups, void* stream)
{
    if ((!x || !y || !y_groups) && n) return fail_invalid("pxh_axpy_norm: null pointer");
    if (has_groups(y, n) && aligned16(x))
        return launch_stream_groups("pxh_axpy_norm", n, 12, AxpyOp{ x, y, alpha }, static_cast<float2*>(y_groups),
                                    as_stream(stream));
    const int rc = pxh_axpy(n, alpha, x, y, stream);
    return rc ? rc : pxh_norm_groups(y, n, y_groups, stream);
}

int pxh_shortcut_backward_norm(float* delta, const float* pre_activation, float* from_delta, float* grad, size_t n,
                               float alpha, float beta, int activation, int first, void* grad_groups, void* stream)
{
    if ((!grad || !grad_groups) && n) return fail_invalid("pxh_shortcut_backward_norm: grad and its group buffer are required");
    const bool flat = has_groups(grad, n) && aligned16(delta) && aligned16(pre_activation) && aligned16(from_delta);
    if (!flat) {
        const int rc = first ? pxh_shortcut_backward_first(delta, pre_activation, from_delta, grad, n, alpha, beta,
                                                           activation, stream)
                             : pxh_shortcut_backward(delta, pre_activation, from_delta, grad, n, alpha, beta,
                                                     activation, stream);
        return rc ? rc : pxh_norm_groups(grad, n, grad_groups, stream);
    }
    if ((!delta || !from_delta) && n) return fail_invalid("pxh_shortcut_backward_norm: null pointer");
    if (activation != PXH_LINEAR && !pre_activation && n)
        return fail_invalid("pxh_shortcut_backward_norm: pre_activation is required for a non-linear activation");
    if (first && from_delta == grad && n)
        return fail_invalid("pxh_shortcut_backward_norm: from_delta and grad must be distinct when both are overwritten");
    int rc = PXH_OK;
    float2* groups = static_cast<float2*>(grad_groups);
    const bool known = dispatch_activation(activation, [&]<int ACT>() {
        if (first)
            rc = launch_stream_groups("pxh_shortcut_backward_norm", n, 12,
                                      ShortcutBackwardOp<ACT, true>{ delta, pre_activation, from_delta, grad, alpha, beta },
                                      groups, as_stream(stream));
        else
            rc = launch_stream_groups("pxh_shortcut_backward_norm", n, 20,
                                      ShortcutBackwardOp<ACT>{ delta, pre_activation, from_delta, grad, alpha, beta },
                                      groups, as_stream(stream));
    });
    if (!known) return fail_invalid("pxh_shortcut_backward_norm: unknown activation %d", activation);
    return rc;
}

size_t pxh_rescale_workspace_bytes(void)
{
    return kNormBlocks * sizeof(double2);      // partial sums and peaks
}

namespace {
// `groups`: the group sums a kernel left when it wrote x, or null to read x for them.
int rescale_clip(const char* who, float* x, size_t n, float threshold, float clip, float* norm_out,
                 const float2* groups, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!x && n) return fail_invalid("%s: null pointer", who);
    if (n == 0) return PXH_OK;
    const bool rescale = threshold > 0.0f || norm_out != nullptr;
    if (!rescale && !(clip > 0.0f)) return PXH_OK;
    void* ws = nullptr;
    int rc = resolve_workspace(workspace, workspace_bytes, pxh_rescale_workspace_bytes(), &ws, as_stream(stream));
    if (rc) return rc;
    double2* partial = static_cast<double2*>(ws);
    hipStream_t s = as_stream(stream);
    const bool vec = has_groups(x, n);
    const int v = vec ? 4 : 1;
    // a tensor past the last-level cache gains nothing from being kept for the next pass
    const bool nt = vec && n * 4 >= kStreamingBytes;
    // the reduction also finds the largest magnitude, which tells whether the clamp can move anything
    const size_t per_step = static_cast<size_t>(kBlock) * v * kNormLoads;
    const size_t want = (n + per_step - 1) / per_step;
    const int blocks = static_cast<int>(want < static_cast<size_t>(kNormBlocks) ? want : kNormBlocks);
    if (vec && groups) {
        const size_t n_groups = (n + kGroupValues - 1) / kGroupValues;
        hipLaunchKernelGGL(norm_chains_kernel, dim3(grid_for(static_cast<size_t>(blocks) * kChains, kBlock)),
                           dim3(kBlock), 0, s, groups, n_groups, static_cast<uint32_t>(blocks), partial);
    }
    else if (nt) hipLaunchKernelGGL((sumsq_partial_kernel<4, true>), dim3(blocks), dim3(kBlock), 0, s, x, n, partial);
    else if (vec) hipLaunchKernelGGL((sumsq_partial_kernel<4, false>), dim3(blocks), dim3(kBlock), 0, s, x, n, partial);
    else hipLaunchKernelGGL((sumsq_partial_kernel<1, false>), dim3(blocks), dim3(kBlock), 0, s, x, n, partial);
    rc = check_launch(who);
    if (rc) return rc;
    // only the norm asked for: one workgroup adds up the partials and writes it
    const dim3 grid(threshold > 0.0f || clip > 0.0f ? static_cast<unsigned>(blocks) : 1u);
    if (nt) hipLaunchKernelGGL((rescale_clip_kernel<4, true>), grid, dim3(kBlock), 0, s, x, n, partial, blocks,
                               threshold, clip, norm_out);
    else if (vec) hipLaunchKernelGGL((rescale_clip_kernel<4, false>), grid, dim3(kBlock), 0, s, x, n, partial, blocks,
                                     threshold, clip, norm_out);
    else hipLaunchKernelGGL((rescale_clip_kernel<1, false>), grid, dim3(kBlock), 0, s, x, n, partial, blocks,
                            threshold, clip, norm_out);
    return check_launch(who);
}
}  // namespace

int pxh_rescale_clip(float* x, size_t n, float threshold, float clip, float* norm_out, void* workspace,
                     size_t workspace_bytes, void* stream)
{
    return rescale_clip("pxh_rescale_clip", x, n, threshold, clip, norm_out, nullptr, workspace, workspace_bytes, stream);
}

int pxh_rescale_clip_from_groups(float* x, size_t n, float threshold, float clip, float* norm_out, const void* groups,
                                 void* workspace, size_t workspace_bytes, void* stream)
{
    if (!groups && n) return fail_invalid("pxh_rescale_clip_from_groups: null group buffer");
    return rescale_clip("pxh_rescale_clip_from_groups", x, n, threshold, clip, norm_out,
                        static_cast<const float2*>(groups), workspace, workspace_bytes, stream);
}

int pxh_shortcut_backward_clipped(float* delta, const float* pre_activation, float* from_delta, float* grad, size_t n,
                                  float alpha, float beta, int activation, int first, float threshold, float clip,
                                  float* norm_out, void* workspace, size_t workspace_bytes, void* stream)
{
    const char* who = "pxh_shortcut_backward_clipped";
    if ((!delta || !from_delta) && n) return fail_invalid("%s: null pointer", who);
    if (activation != PXH_LINEAR && !pre_activation && n)
        return fail_invalid("%s: pre_activation is required for a non-linear activation", who);
    if (first && from_delta == grad && n)
        return fail_invalid("%s: from_delta and grad must be distinct when both are overwritten", who);
    if ((delta == from_delta || delta == grad) && n) return fail_invalid("%s: delta must be a tensor of its own", who);
    if (activation < PXH_LEAKY || activation > PXH_TANH) return fail_invalid("%s: unknown activation %d", who, activation);
    if (n == 0) return PXH_OK;
    const bool helpers = threshold > 0.0f || clip > 0.0f || norm_out != nullptr;
    const bool fused = helpers && first && activation == PXH_LINEAR && has_groups(delta, n) && aligned16(from_delta) &&
                       aligned16(grad);
    if (!fused) {
        // the two calls one after the other: the accumulating form (what it adds to cannot be taken back), a
        // non-linear shortcut (its backward rewrites the delta), tensors without a 128-bit walk
        int rc = helpers ? rescale_clip(who, delta, n, threshold, clip, norm_out, nullptr, workspace, workspace_bytes, stream)
                         : PXH_OK;
        if (rc) return rc;
        return first ? pxh_shortcut_backward_first(delta, pre_activation, from_delta, grad, n, alpha, beta, activation, stream)
                     : pxh_shortcut_backward(delta, pre_activation, from_delta, grad, n, alpha, beta, activation, stream);
    }
    void* ws = nullptr;
    int rc = resolve_workspace(workspace, workspace_bytes, pxh_rescale_workspace_bytes(), &ws, as_stream(stream));
    if (rc) return rc;
    double2* partial = static_cast<double2*>(ws);
    hipStream_t s = as_stream(stream);
    const bool nt = n * (grad ? 12 : 8) >= kStreamingBytes;
    // the workgroups and the walk of pxh_rescale_clip's own passes: the same partial sums, the same norm
    const size_t per_step = static_cast<size_t>(kBlock) * 4 * kNormLoads;
    const size_t want = (n + per_step - 1) / per_step;
    const int blocks = static_cast<int>(want < static_cast<size_t>(kNormBlocks) ? want : kNormBlocks);
    const ShortcutFirstSink sink{ from_delta, grad, alpha, beta };
    if (nt) hipLaunchKernelGGL((sumsq_sink_kernel<true, ShortcutFirstSink>), dim3(blocks), dim3(kBlock), 0, s, delta, n,
                               partial, sink);
    else hipLaunchKernelGGL((sumsq_sink_kernel<false, ShortcutFirstSink>), dim3(blocks), dim3(kBlock), 0, s, delta, n,
                            partial, sink);
    rc = check_launch(who);
    if (rc) return rc;
    const dim3 grid(threshold > 0.0f || clip > 0.0f ? static_cast<unsigned>(blocks) : 1u);
    if (nt) hipLaunchKernelGGL((rescale_clip_sink_kernel<true, ShortcutFirstSink>), grid, dim3(kBlock), 0, s, delta, n,
                               partial, blocks, threshold, clip, norm_out, sink);
    else hipLaunchKernelGGL((rescale_clip_sink_kernel<false, ShortcutFirstSink>), grid, dim3(kBlock), 0, s, delta, n,
                            partial, blocks, threshold, clip, norm_out, sink);
    return check_launch(who);
}

size_t pxh_rescale_multi_workspace_bytes(void)
{
    return static_cast<size_t>(kRescaleTensors) * kNormBlocks * sizeof(double2);
}

int pxh_rescale_clip_multi(int count, float* const* x, const size_t* n, float threshold, float clip, float* norms,
                           void* workspace, size_t workspace_bytes, void* stream)
{
    if (count < 0 || (count && (!x || !n))) return fail_invalid("pxh_rescale_clip_multi: bad argument");
    const bool rescale = threshold > 0.0f || norms != nullptr;
    if (!rescale && !(clip > 0.0f)) return PXH_OK;
    void* ws = nullptr;
    int rc = resolve_workspace(workspace, workspace_bytes, pxh_rescale_multi_workspace_bytes(), &ws, as_stream(stream));
    if (rc) return rc;
    double2* partial = static_cast<double2*>(ws);
    hipStream_t s = as_stream(stream);
    for (int begin = 0; begin < count; begin += kRescaleTensors) {
        RescaleTable t{};
        const int part = count - begin < kRescaleTensors ? count - begin : kRescaleTensors;
        uint32_t blocks = 0;
        for (int i = 0; i < part; ++i) {
            // an empty tensor keeps its place in the table with no workgroup of its own (its norm stays unwritten)
            float* ptr = x[begin + i];
            const size_t len = n[begin + i];
            if (!ptr && len) return fail_invalid("pxh_rescale_clip_multi: null pointer for tensor %d", begin + i);
            const bool vec = aligned16(ptr) && len % 4 == 0;
            const size_t per_step = static_cast<size_t>(kBlock) * (vec ? 4 : 1) * kNormLoads;
            const size_t want = (len + per_step - 1) / per_step;
            t.x[i] = ptr;
            t.n[i] = len;
            t.first_block[i] = blocks;
            if (vec) t.vector_mask |= 1u << i;
            if (vec && len * 4 >= kStreamingBytes) t.past_cache_mask |= 1u << i;
            blocks += static_cast<uint32_t>(want < static_cast<size_t>(kNormBlocks) ? want : kNormBlocks);
        }
        t.first_block[part] = blocks;
        t.count = part;
        t.norms = norms;
        t.first_tensor = begin;
        if (blocks == 0) continue;
        hipLaunchKernelGGL(multi_sumsq_kernel, dim3(blocks), dim3(kBlock), 0, s, t, partial);
        rc = check_launch("pxh_rescale_clip_multi");
        if (rc) return rc;
        hipLaunchKernelGGL(multi_rescale_kernel, dim3(blocks), dim3(kBlock), 0, s, t, partial, threshold, clip);
        rc = check_launch("pxh_rescale_clip_multi");
        if (rc) return rc;
    }
    return PXH_OK;
}

int pxh_adam(int n, float* x, const float* m, const float* v, float beta1, float beta2, float rate, float eps, int t,
             void* stream)
{
    if (n < 0 || ((!x || !m || !v) && n)) return fail_invalid("pxh_adam: bad argument");
    // bias corrections formed on the host in fp32, as powf(beta, t)
    const float c1 = 1.0f - powf(beta1, static_cast<float>(t));
    const float c2 = 1.0f - powf(beta2, static_cast<float>(t));
    return launch_stream("pxh_adam", static_cast<size_t>(n), aligned16(x) && aligned16(m) && aligned16(v), 16,
                         AdamStepOp{ x, m, v, c1, c2, rate, eps }, as_stream(stream));
}

int pxh_adam_update(size_t n, float* w, float* d, float* m, float* v, int batch, int t, float lr, float beta1,
                    float beta2, float eps, float decay, int apply_decay, void* stream)
{
    if ((!w || !d || !m || !v) && n) return fail_invalid("pxh_adam_update: null pointer");
    if (batch <= 0) return fail_invalid("pxh_adam_update: batch must be positive");
    if (t < 1) return fail_invalid("pxh_adam_update: t must be at least 1 (the update count is pre-incremented)");
    if (apply_decay < 0 || apply_decay > 2)
        return fail_invalid("pxh_adam_update: apply_decay is 0 (none), 1 (folded into the update) or 2 (decoupled)");
    AdamUpdateOp op;
    op.w = w; op.d = d; op.m = m; op.v = v;
    op.inv_batch = 1.0f / static_cast<float>(batch);
    op.neg_decay = -decay;
    op.neg_lr_decay = -(lr * decay);
    op.beta1 = beta1; op.beta2 = beta2;
    op.a1 = 1.0f - beta1; op.a2 = 1.0f - beta2;
    op.c1 = 1.0f - powf(beta1, static_cast<float>(t));
    op.c2 = 1.0f - powf(beta2, static_cast<float>(t));
    op.lr = lr; op.eps = eps; op.apply_decay = apply_decay;
    return launch_stream("pxh_adam_update", n, aligned16(w) && aligned16(d) && aligned16(m) && aligned16(v), 32, op,
                         as_stream(stream), kStreamingBytes, true);
}

int pxh_adam_update_multi(int count, float* const* w, float* const* d, float* const* m, float* const* v, const size_t* n,
                          const int* apply_decay, int batch, int t, float lr, float beta1, float beta2, float eps,
                          float decay, void* stream)
{
    if (count < 0 || (count && (!w || !d || !m || !v || !n))) return fail_invalid("pxh_adam_update_multi: bad argument");
    if (batch <= 0) return fail_invalid("pxh_adam_update_multi: batch must be positive");
    if (t < 1) return fail_invalid("pxh_adam_update_multi: t must be at least 1 (the update count is pre-incremented)");
    AdamUpdateOp op{};
    op.inv_batch = 1.0f / static_cast<float>(batch);
    op.neg_decay = -decay;
    op.beta1 = beta1; op.beta2 = beta2;
    op.a1 = 1.0f - beta1; op.a2 = 1.0f - beta2;
    op.c1 = 1.0f - powf(beta1, static_cast<float>(t));
    op.c2 = 1.0f - powf(beta2, static_cast<float>(t));
    op.lr = lr; op.eps = eps;
    float* const* const buffers[4] = { w, d, m, v };
    return launch_multi<4>("pxh_adam_update_multi", count, buffers, n, apply_decay, 32, AdamMaker{ op }, as_stream(stream));
}

int pxh_fill_f32_multi(int count, float* const* x, const size_t* n, float value, void* stream)
{
    if (count < 0 || (count && (!x || !n))) return fail_invalid("pxh_fill_f32_multi: bad argument");
    float* const* const buffers[4] = { x, nullptr, nullptr, nullptr };
    // a fill streams past the caches from the size on that the single call does
    return launch_multi<1>("pxh_fill_f32_multi", count, buffers, n, nullptr, 4, FillMaker{ value }, as_stream(stream),
                           kFillStreamingBytes);
}

// ---------------------------------------------------------------- tensor tables
struct pxh_tensor_table {
    int device;
    int count, streams;
    unsigned long long total_elems;
    uint32_t blocks, norm_blocks;
    void* memory;
    pxh::TableView view;
};

int pxh_tensor_table_create(int count, int streams, float* const* buffers, const size_t* n, const int* apply_decay,
                            pxh_tensor_table** table)
{
    if (!table) return fail_invalid("pxh_tensor_table_create: null pointer");
    *table = nullptr;
    if (count < 0 || (count && (!buffers || !n))) return fail_invalid("pxh_tensor_table_create: bad argument");
    if (streams != 1 && streams != 2 && streams != 4)
        return fail_invalid("pxh_tensor_table_create: 1, 2 or 4 buffers per tensor (got %d)", streams);
    // empty tensors take no part: they are left out of the table
    std::vector<TensorRecord> records;
    std::vector<uint32_t> first_block, first_norm_block;
    unsigned long long blocks = 0, norm_blocks = 0;
    for (int i = 0; i < count; ++i) {
        if (n[i] == 0) continue;
        TensorRecord r{};
        bool aligned = true;
        for (int k = 0; k < streams; ++k) {
            float* ptr = buffers[static_cast<size_t>(k) * count + i];
            if (!ptr) return fail_invalid("pxh_tensor_table_create: null pointer for tensor %d", i);
            aligned = aligned && aligned16(ptr);
            r.stream[k] = ptr;
        }
        r.n = n[i];
        r.decay = apply_decay && apply_decay[i] ? 1u : 0u;
        r.vector = aligned ? 1u : 0u;
        r.norm_vector = aligned16(r.stream[0]) && n[i] % 4 == 0 ? 1u : 0u;
        records.push_back(r);
        first_block.push_back(static_cast<uint32_t>(blocks));
        first_norm_block.push_back(static_cast<uint32_t>(norm_blocks));
        blocks += (n[i] + kTablePerBlock - 1) / kTablePerBlock;
        // the norm pass of the single call: at most kNormBlocks workgroups, each a whole step of loads
        const size_t per_step = static_cast<size_t>(kBlock) * (r.norm_vector ? 4 : 1) * kNormLoads;
        const size_t want = (n[i] + per_step - 1) / per_step;
        norm_blocks += want < static_cast<size_t>(kNormBlocks) ? want : kNormBlocks;
    }
    if (records.size() > static_cast<size_t>(kMaxTableTensors)) {
        set_error("pxh_tensor_table_create: %zu tensors; a table holds %d at most", records.size(), kMaxTableTensors);
        return PXH_ERR_UNSUPPORTED;
    }
    if (blocks > 0x7fffffffull) {
        set_error("pxh_tensor_table_create: more than 2^31 workgroups in one launch");
        return PXH_ERR_UNSUPPORTED;
    }
    first_block.push_back(static_cast<uint32_t>(blocks));
    first_norm_block.push_back(static_cast<uint32_t>(norm_blocks));

    auto* t = new (std::nothrow) pxh_tensor_table{};
    if (!t) return fail_invalid("pxh_tensor_table_create: out of host memory");
    t->count = static_cast<int>(records.size());
    t->streams = streams;
    for (const TensorRecord& r: records) t->total_elems += r.n;
    t->blocks = static_cast<uint32_t>(blocks);
    t->norm_blocks = static_cast<uint32_t>(norm_blocks);
    if (hipGetDevice(&t->device) != hipSuccess) t->device = -1;
    if (t->count == 0) {
        *table = t;
        return PXH_OK;
    }
    // one allocation: records | first workgroups | first norm workgroups | partial sums of the norm pass
    const auto align = [](size_t b) { return (b + 255) & ~static_cast<size_t>(255); };
    const size_t rec_bytes = align(records.size() * sizeof(TensorRecord));
    const size_t first_bytes = align(first_block.size() * sizeof(uint32_t));
    const size_t partial_bytes = align(static_cast<size_t>(norm_blocks) * sizeof(double2));
    const size_t total = rec_bytes + 2 * first_bytes + partial_bytes;
    hipError_t e = hipMalloc(&t->memory, total);
    if (e != hipSuccess) {
        set_error("pxh_tensor_table_create: hipMalloc(%zu): %s", total, hipGetErrorString(e));
        delete t;
        return static_cast<int>(e);
    }
    char* base = static_cast<char*>(t->memory);
    std::vector<char> image(rec_bytes + 2 * first_bytes, 0);
    std::memcpy(image.data(), records.data(), records.size() * sizeof(TensorRecord));
    std::memcpy(image.data() + rec_bytes, first_block.data(), first_block.size() * sizeof(uint32_t));
    std::memcpy(image.data() + rec_bytes + first_bytes, first_norm_block.data(), first_norm_block.size() * sizeof(uint32_t));
    e = hipMemcpy(base, image.data(), image.size(), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        set_error("pxh_tensor_table_create: upload: %s", hipGetErrorString(e));
        (void) hipFree(t->memory);
        delete t;
        return static_cast<int>(e);
    }
    t->view.records = reinterpret_cast<const TensorRecord*>(base);
    t->view.first_block = reinterpret_cast<const uint32_t*>(base + rec_bytes);
    t->view.first_norm_block = reinterpret_cast<const uint32_t*>(base + rec_bytes + first_bytes);
    t->view.partial = reinterpret_cast<double2*>(base + rec_bytes + 2 * first_bytes);
    t->view.count = t->count;
    *table = t;
    return PXH_OK;
}

void pxh_tensor_table_destroy(pxh_tensor_table* table)
{
    if (!table) return;
    if (table->memory) (void) hipFree(table->memory);
    delete table;
}

int pxh_tensor_table_count(const pxh_tensor_table* table) { return table ? table->count : 0; }

extern "C++" {
namespace {
template<typename Maker>
int launch_table(const char* who, const pxh_tensor_table* table, int streams_needed, int bytes_per_elem, const Maker& make,
                 void* stream, size_t streaming_from = kStreamingBytes)
{
    if (!table) return fail_invalid("%s: null table", who);
    if (table->streams < streams_needed)
        return fail_invalid("%s: the table holds %d buffers per tensor, %d are needed", who, table->streams, streams_needed);
    if (table->count == 0) return PXH_OK;
    // the tensors of a table are walked in one sweep: whether that sweep outgrows the last-level cache is a
    // matter of all of them together, not of each one's size
    const bool past_cache = table->total_elems * static_cast<unsigned long long>(bytes_per_elem) >= streaming_from;
    const unsigned long long streaming_elems = past_cache ? 0ull : ~0ull;
    hipLaunchKernelGGL((table_stream_kernel<Maker>), dim3(table->blocks), dim3(kBlock), 0, as_stream(stream), table->view,
                       make, streaming_elems);
    return check_launch(who);
}
}  // namespace
}  // extern "C++"

int pxh_adam_update_table(const pxh_tensor_table* table, int batch, int t, float lr, float beta1, float beta2, float eps,
                          float decay, void* stream)
{
    if (batch <= 0) return fail_invalid("pxh_adam_update_table: batch must be positive");
    if (t < 1) return fail_invalid("pxh_adam_update_table: t must be at least 1 (the update count is pre-incremented)");
    AdamUpdateOp op{};
    op.inv_batch = 1.0f / static_cast<float>(batch);
    op.neg_decay = -decay;
    op.beta1 = beta1; op.beta2 = beta2;
    op.a1 = 1.0f - beta1; op.a2 = 1.0f - beta2;
    op.c1 = 1.0f - powf(beta1, static_cast<float>(t));
    op.c2 = 1.0f - powf(beta2, static_cast<float>(t));
    op.lr = lr; op.eps = eps;
    return launch_table("pxh_adam_update_table", table, 4, 32, AdamFromRecord{ op }, stream);
}

int pxh_sgd_update_table(const pxh_tensor_table* table, int batch, float lr, float momentum, float decay, void* stream)
{
    if (batch <= 0) return fail_invalid("pxh_sgd_update_table: batch must be positive");
    const SgdUpdateOp op{ nullptr, nullptr, -decay * static_cast<float>(batch), lr / static_cast<float>(batch), momentum, 0 };
    return launch_table("pxh_sgd_update_table", table, 2, 16, SgdFromRecord{ op }, stream);
}

int pxh_fill_f32_table(const pxh_tensor_table* table, float value, void* stream)
{
    return launch_table("pxh_fill_f32_table", table, 1, 4, FillFromRecord{ value }, stream, kFillStreamingBytes);
}

int pxh_rescale_clip_table(const pxh_tensor_table* table, float threshold, float clip, float* norms, void* stream)
{
    if (!table) return fail_invalid("pxh_rescale_clip_table: null table");
    const bool rescale = threshold > 0.0f || norms != nullptr;
    if ((!rescale && !(clip > 0.0f)) || table->count == 0) return PXH_OK;
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(table_sumsq_kernel, dim3(table->norm_blocks), dim3(kBlock), 0, s, table->view);
    int rc = check_launch("pxh_rescale_clip_table");
    if (rc) return rc;
    hipLaunchKernelGGL(table_rescale_kernel, dim3(table->norm_blocks), dim3(kBlock), 0, s, table->view, threshold, clip,
                       norms);
    return check_launch("pxh_rescale_clip_table");
}

int pxh_sgd_update_multi(int count, float* const* w, float* const* d, const size_t* n, const int* apply_decay, int batch,
                         float lr, float momentum, float decay, void* stream)
{
    if (count < 0 || (count && (!w || !d || !n))) return fail_invalid("pxh_sgd_update_multi: bad argument");
    if (batch <= 0) return fail_invalid("pxh_sgd_update_multi: batch must be positive");
    const SgdUpdateOp op{ nullptr, nullptr, -decay * static_cast<float>(batch), lr / static_cast<float>(batch), momentum, 0 };
    float* const* const buffers[4] = { w, d, nullptr, nullptr };
    return launch_multi<2>("pxh_sgd_update_multi", count, buffers, n, apply_decay, 16, SgdMaker{ op }, as_stream(stream));
}

int pxh_debug_stream_mix(int reads, int writes, size_t n, const float* const* in, float* const* out, void* stream)
{
    if (reads < 1 || reads > 4 || writes < 1 || writes > 4 || !in || !out || n % 4)
        return fail_invalid("pxh_debug_stream_mix: 1..4 streams each way, n a multiple of 4");
    for (int i = 0; i < reads; ++i)
        if (!in[i] || !aligned16(in[i])) return fail_invalid("pxh_debug_stream_mix: bad input pointer %d", i);
    for (int i = 0; i < writes; ++i)
        if (!out[i] || !aligned16(out[i])) return fail_invalid("pxh_debug_stream_mix: bad output pointer %d", i);
    hipStream_t s = as_stream(stream);
    switch (reads * 10 + writes) {
    case 11: return launch_mix<1, 1>(n, in, out, s);
    case 12: return launch_mix<1, 2>(n, in, out, s);
    case 13: return launch_mix<1, 3>(n, in, out, s);
    case 14: return launch_mix<1, 4>(n, in, out, s);
    case 21: return launch_mix<2, 1>(n, in, out, s);
    case 22: return launch_mix<2, 2>(n, in, out, s);
    case 23: return launch_mix<2, 3>(n, in, out, s);
    case 24: return launch_mix<2, 4>(n, in, out, s);
    case 31: return launch_mix<3, 1>(n, in, out, s);
    case 32: return launch_mix<3, 2>(n, in, out, s);
    case 33: return launch_mix<3, 3>(n, in, out, s);
    case 34: return launch_mix<3, 4>(n, in, out, s);
    case 41: return launch_mix<4, 1>(n, in, out, s);
    case 42: return launch_mix<4, 2>(n, in, out, s);
    case 43: return launch_mix<4, 3>(n, in, out, s);
    default: return launch_mix<4, 4>(n, in, out, s);
    }
}

}
