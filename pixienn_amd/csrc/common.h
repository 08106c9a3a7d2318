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
// Per-device scratch the library owns, grown on demand and kept until exit.
void* library_workspace(size_t bytes);
// Picks the caller's workspace when given (checking its size), else the library's.
int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out);

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
__device__ __forceinline__ float softplus_apply(float x)
{
    if (x > 20.0f) return x;
    if (x < -20.0f) return expf(x);
    return logf(expf(x) + 1.0f);
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
    return tanh_softplus_from_exp(expf(x));
}

// Forward mish without branches.  exp stays the accurate one: u = fl(exp(x) + 1) is where the CPU
// chain loses its bits for negative x, so a last-place difference in exp(x) can show as 1e-5 of
// the result (measured with the hardware exp2: 3 elements per million beyond 1e-5).  The division
// is a hardware reciprocal and a multiply, 2 ulp.
__device__ __forceinline__ float mish_apply(float x)
{
    const float e = expf(x);
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
    // logistic and swish: the accurate exp, then a hardware reciprocal (1 ulp) in place of the division
    else if constexpr (ACT == PXH_LOGISTIC) return __builtin_amdgcn_rcpf(1.0f + expf(-x));
    else if constexpr (ACT == PXH_MISH) return mish_apply(x);
    else if constexpr (ACT == PXH_RELU) return x > 0.0f ? x : 0.0f;
    else if constexpr (ACT == PXH_SOFTPLUS) return softplus_apply(x);
    else if constexpr (ACT == PXH_SWISH) return x * __builtin_amdgcn_rcpf(1.0f + expf(-1.0f * x));
    else return tanhf(x);
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

inline unsigned grid_for(size_t items, size_t per_block)
{
    return static_cast<unsigned>((items + per_block - 1) / per_block);
}

}  // namespace pxh
