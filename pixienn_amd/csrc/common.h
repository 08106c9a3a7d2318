// Shared host/device helpers for the gfx950 layer kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "../../include/pixienn_hip.h"

namespace pxh {

constexpr int kWave = 64;          // CDNA wavefront
constexpr int kBlock = 256;        // 4 waves per workgroup

// ---------------------------------------------------------------- errors
void set_error(const char* fmt, ...);
int fail_invalid(const char* fmt, ...);
int check_launch(const char* what);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- workspace
// Picks the caller's workspace when given (checking its size), else the per-device buffer the
// library owns, which grows on demand (never while `stream` is being captured) and is kept until exit.
int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out, hipStream_t stream);

// ---------------------------------------------------------------- fast division
// q = n / d for 0 <= n < 2^31 by a multiply-high and a shift (d >= 1).
struct FastDiv {
    uint32_t d, m, s;
    FastDiv() : d(1), m(0), s(0) {}
    explicit FastDiv(uint32_t div) : d(div)
    {
        s = 0;
        while ((1ull << s) < div) ++s;
        m = static_cast<uint32_t>(((1ull << 32) * ((1ull << s) - div)) / div + 1);
    }
    __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const
    {
#if defined(__HIP_DEVICE_COMPILE__)
        uint32_t t = __umulhi(n, m);
#else
        uint32_t t = static_cast<uint32_t>((static_cast<uint64_t>(n) * m) >> 32);
#endif
        return (t + n) >> s;
    }
    __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const
    {
        q = div(n);
        r = n - q * d;
    }
};

// ---------------------------------------------------------------- activations (device)
// The arithmetic follows the CPU functors operation by operation (fp32, no contraction).
// exp(x) to about a unit in the last place around the hardware's exp2: x * log2(e) is formed to twice
// the working precision (the fma recovers the product's rounding error, a second term carries the low
// bits of log2(e)), split into its integer part and a fraction in [-0.5, 0.5], and only the fraction
// goes through exp2.  No range checks: ldexp saturates to 0 and infinity by itself.
__device__ __forceinline__ float exp_by_exp2(float x)
{
    const float hi = 0x1.715476p+0f, lo = 0x1.4ae0c0p-26f;      // log2(e) = hi + lo
    const float p = x * hi;
    const float err = fmaf(x, lo, fmaf(x, hi, -p));
    const float n = rintf(p);
    const float f = (p - n) + err;
    return ldexpf(__builtin_amdgcn_exp2f(f), static_cast<int>(n));
}

// exp(x) rounded to nearest, through a double-precision evaluation (argument reduction by ln 2,
// Taylor polynomial of degree 10 on |r| <= 0.35: 2.4e-13 relative, so the conversion to float rounds
// as the exact value would except within 2e-6 of a tie).
__device__ __forceinline__ float exp_nearest(float x)
{
    const double xd = static_cast<double>(x);
    const double k = rint(xd * 1.4426950408889634);
    double r = fma(-k, 0.6931471805599453, xd);
    r = fma(-k, 2.3190468138462996e-17, r);
    double p = 1.0 / 3628800.0;
    p = fma(p, r, 1.0 / 362880.0);
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return static_cast<float>(ldexp(p, static_cast<int>(k)));
}

// e = exp(x) for the chains that go on with u = float(e + 1) (softplus and everything built on it).
// Below x = -4.4 (e < 0.012) one unit of u = 1.2e-7 is more than 1e-5 of e, and the CPU result moves
// by that whole unit -- up to 0.4 % of its value -- when e is one unit in ITS last place off: there e
// has to be the correctly rounded value the host's libm returns (measured with a 1-ulp exp: 25
// elements per million of x in [-10.5, -4.4] off by up to 1e-3).  Such arguments are rare in a network
// (a pre-activation 4 sigma below zero), so the double-precision path costs a wave only now and
// then; elsewhere one unit in the last place is plenty and the short form is used.
__device__ __forceinline__ bool one_plus_exp_is_sensitive(float x) { return x < -4.4f && x >= -20.0f; }

__device__ __forceinline__ float exp_before_one_plus(float x)
{
    float e = exp_by_exp2(x);
    if (one_plus_exp_is_sensitive(x)) e = exp_nearest(x);
    return e;
}

__device__ __forceinline__ float softplus_apply(float x)
{
    if (x > 20.0f) return x;
    if (x < -20.0f) return expf(x);
    return logf(exp_before_one_plus(x) + 1.0f);
}

__device__ __forceinline__ float softplus_grad(float x)
{
    if (x > 20.0f) return 1.0f;
    if (x < -20.0f) return expf(x);
    return 1.0f / (1.0f + expf(-x));
}

// tanh(softplus(x)) for |x| <= 20.  The CPU functor evaluates tanhf(logf(u)) with
// u = float(expf(x) + 1); tanh(log u) = (u*u - 1)/(u*u + 1) exactly, and (u - 1) is exact in
// fp32, so the same rounded u gives the same value to a few ulp with one exp and one division
// instead of exp + log + tanh.
__device__ __forceinline__ float tanh_softplus_from_exp(float e)
{
    const float u = e + 1.0f;
    const float num = (u - 1.0f) * (u + 1.0f);
    const float den = u * u + 1.0f;
    return num / den;
}

__device__ __forceinline__ float tanh_softplus_mid(float x)
{
    return tanh_softplus_from_exp(exp_before_one_plus(x));
}

// Forward mish: one exp (see exp_before_one_plus), the division as a hardware reciprocal and a
// multiply (2 ulp), the two tails by selection.
template<bool QUICK = false>
__device__ __forceinline__ float mish_apply(float x)
{
    const float e = QUICK ? exp_by_exp2(x) : exp_before_one_plus(x);
    const float u = e + 1.0f;
    const float num = (u - 1.0f) * (u + 1.0f);
    const float den = u * u + 1.0f;
    const float mid = num * __builtin_amdgcn_rcpf(den);
    // x > 20: tanhf(softplus) is 1.0f; x < -20: tanhf(s) is s = exp(x) for s < 2.1e-9
    const float t = x < -20.0f ? e : mid;
    return x > 20.0f ? x : x * t;
}

__device__ __forceinline__ float mish_grad(float x)
{
    if (x > 20.0f) return 1.0f;              // (1 - 1*1)*1*x + 1
    float tsp, gsp;
    if (x < -20.0f) {
        tsp = expf(x);
        gsp = tsp;
    } else {
        tsp = tanh_softplus_mid(x);
        gsp = 1.0f / (1.0f + expf(-x));
    }
    const float gtsp = (1.0f - tsp * tsp) * gsp;
    return x * gtsp + tsp;
}

template<int ACT>
__device__ __forceinline__ float act_apply(float x)
{
    if constexpr (ACT == PXH_LEAKY) return x > 0.0f ? x : 0.1f * x;
    else if constexpr (ACT == PXH_LINEAR) return x;
    else if constexpr (ACT == PXH_LOGGY) return 2.0f / (1.0f + expf(-x)) - 1.0f;
    // logistic and swish: the short exp (a unit in the last place, as for mish) and a hardware reciprocal
    // (1 ulp) in place of the division: the sum 1 + e absorbs e's last place wherever the result is not
    // already proportional to 1 / e
    else if constexpr (ACT == PXH_LOGISTIC) return __builtin_amdgcn_rcpf(1.0f + exp_by_exp2(-x));
    else if constexpr (ACT == PXH_MISH) return mish_apply<false>(x);
    else if constexpr (ACT == PXH_RELU) return x > 0.0f ? x : 0.0f;
    else if constexpr (ACT == PXH_SOFTPLUS) return softplus_apply(x);
    else if constexpr (ACT == PXH_SWISH) return x * __builtin_amdgcn_rcpf(1.0f + exp_by_exp2(-1.0f * x));
    else return tanhf(x);
}

// V values at once.  For mish the short exp goes everywhere first and the values whose argument is
// in the sensitive range are redone, behind ONE branch for the whole wave instead of one per value:
// the same results as act_apply value by value.
template<int ACT, int V>
__device__ __forceinline__ void act_apply_n(const float (&pre)[V], float (&out)[V])
{
    if constexpr (ACT == PXH_MISH) {
        bool any = false;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            out[k] = mish_apply<true>(pre[k]);
            any = any | one_plus_exp_is_sensitive(pre[k]);
        }
        if (__ballot(any)) {
#pragma unroll
            for (int k = 0; k < V; ++k)
                if (one_plus_exp_is_sensitive(pre[k])) out[k] = mish_apply<false>(pre[k]);
        }
    } else {
#pragma unroll
        for (int k = 0; k < V; ++k) out[k] = act_apply<ACT>(pre[k]);
    }
}

template<int ACT>
__device__ __forceinline__ float act_grad(float x)
{
    if constexpr (ACT == PXH_LEAKY) return x > 0.0f ? 1.0f : 0.1f;
    else if constexpr (ACT == PXH_LINEAR) return 1.0f;
    else if constexpr (ACT == PXH_LOGGY) {
        float y = (x + 1.0f) / 2.0f;
        return 2.0f * (1.0f - y) * y;
    } else if constexpr (ACT == PXH_LOGISTIC) {
        float y = 1.0f / (1.0f + expf(-x));
        return y * (1.0f - y);
    } else if constexpr (ACT == PXH_MISH) {
        return mish_grad(x);
    } else if constexpr (ACT == PXH_RELU) return x > 0.0f ? 1.0f : 0.0f;
    else if constexpr (ACT == PXH_SOFTPLUS) return softplus_grad(x);
    else if constexpr (ACT == PXH_SWISH) {
        float val = 1.0f / (1.0f + expf(-1.0f * x));
        return x * val + 1.0f * val * (1.0f - x * val);
    } else {
        float y = tanhf(x);
        return 1.0f - y * y;
    }
}

// Calls f.template operator()<ACT>() for the runtime activation id; false if unknown.
template<typename F>
inline bool dispatch_activation(int act, F&& f)
{
    switch (act) {
    case PXH_LEAKY: f.template operator()<PXH_LEAKY>(); return true;
    case PXH_LINEAR: f.template operator()<PXH_LINEAR>(); return true;
    case PXH_LOGGY: f.template operator()<PXH_LOGGY>(); return true;
    case PXH_LOGISTIC: f.template operator()<PXH_LOGISTIC>(); return true;
    case PXH_MISH: f.template operator()<PXH_MISH>(); return true;
    case PXH_RELU: f.template operator()<PXH_RELU>(); return true;
    case PXH_SOFTPLUS: f.template operator()<PXH_SOFTPLUS>(); return true;
    case PXH_SWISH: f.template operator()<PXH_SWISH>(); return true;
    case PXH_TANH: f.template operator()<PXH_TANH>(); return true;
    default: return false;
    }
}

// ---------------------------------------------------------------- reductions
// Sum over the 64 lanes of a wavefront; every lane returns the total.
__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// The value of another lane of the same row of 16 (a data-parallel-primitive operand: no trip through
// the LDS crossbar, unlike __shfl).  CTRL: 0xB1 = lane ^ 1, 0x4E = lane ^ 2, 0x141 = 7 - lane within each
// half row, 0x140 = 15 - lane within the row.  All lanes of the wave must be active.
template<int CTRL>
__device__ __forceinline__ float lane_in_row(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float from_lane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Sum over the 64 lanes in one fixed tree -- pairs, quads, eights, rows of 16, then
// (row0 + row1) + (row2 + row3) -- with the same total in every lane.  Four full-rate
// instructions and four lane reads: the form for a sum that is taken once per vector loaded.
// All lanes of the wave must be active.
__device__ __forceinline__ float wave_sum_by_rows(float v)
{
    v += lane_in_row<0xB1>(v);
    v += lane_in_row<0x4E>(v);
    v += lane_in_row<0x141>(v);
    v += lane_in_row<0x140>(v);
    const float r0 = from_lane(v, 0), r1 = from_lane(v, 16), r2 = from_lane(v, 32), r3 = from_lane(v, 48);
    return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ float wave_max_by_rows(float v)
{
    v = fmaxf(v, lane_in_row<0xB1>(v));
    v = fmaxf(v, lane_in_row<0x4E>(v));
    v = fmaxf(v, lane_in_row<0x141>(v));
    v = fmaxf(v, lane_in_row<0x140>(v));
    const float r0 = from_lane(v, 0), r1 = from_lane(v, 16), r2 = from_lane(v, 32), r3 = from_lane(v, 48);
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Sum over a kBlock-thread workgroup through LDS; result valid in thread 0.
// `slots` is LDS of at least kBlock / kWave doubles per concurrently reduced value.
__device__ __forceinline__ double block_sum(double v, double* slots)
{
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    double total = 0.0;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kBlock / kWave; ++w) total += slots[w];
    }
    return total;
}

// ---------------------------------------------------------------- gradient rescale + clip: the decision
// Layer::backward's two helpers on a delta (include/Layer.h:385-397, 479-499 of the reference):
//   norm = |x|_2;  if (norm > 0 && norm > threshold) x *= threshold / norm;  then clamp to +-clip.
// From the sum of squares and the largest magnitude: the norm, the factor, and whether anything can
// change -- a factor other than 1, or a value that the clamp would move.  The scaled magnitudes are at
// most fl(factor * peak) (rounding is monotonic), so a peak within the clamp after scaling means no
// element changes; a NaN anywhere (it shows in the sum) or an infinite peak keeps the rewrite, which
// treats them as the CPU loop does.
struct RescalePlan {
    float norm, factor;
    bool work;      // some value changes
    bool clamps;    // ... and not by the factor alone: the clamp may move one
};

__device__ __forceinline__ RescalePlan plan_from_totals(double total, float peak, float threshold, float clip)
{
    RescalePlan plan;
    plan.norm = static_cast<float>(sqrt(total));
    plan.factor = 1.0f;
    if (threshold > 0.0f && plan.norm > 0.0f && plan.norm > threshold) plan.factor = threshold / plan.norm;
    plan.clamps = clip > 0.0f && (!(plan.factor * peak <= clip) || total != total);
    plan.work = plan.factor != 1.0f || plan.clamps;
    return plan;
}

// One value through the two helpers.
__device__ __forceinline__ float rescaled_clipped(float x, float factor, float clip)
{
    float t = factor == 1.0f ? x : factor * x;
    if (clip > 0.0f) t = fminf(clip, fmaxf(-clip, t));
    return t;
}

inline unsigned grid_for(size_t items, size_t per_block)
{
    return static_cast<unsigned>((items + per_block - 1) / per_block);
}

}  // namespace pxh
