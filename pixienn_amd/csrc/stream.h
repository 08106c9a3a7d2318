// Flat streaming skeleton.
//
// Measured on MI355X with a plain copy kernel: one 128-bit access per stream per lane and many
// small workgroups beat deeper per-lane unrolling (6.2 vs 5.6 TB/s), and non-temporal accesses
// add another 7 % once the tensors no longer fit the 256 MB last-level cache, while they cost
// 10 % on tensors that do fit.  So: kBlock lanes, one vector per lane per stream, and a
// non-temporal variant chosen by the bytes a launch touches.
//
// An operation supplies
//     template<int V> struct Regs;                                     // state between the phases
//     template<int V, bool NT> __device__ void load(size_t e, Regs<V>&) const;   // e = first element
//     template<int V, bool NT> __device__ void finish(size_t e, const Regs<V>&) const;
// V is 4 for the 128-bit path and 1 for the scalar path (unaligned pointers and the n % 4 tail).
#pragma once

#include "common.h"

namespace pxh {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

// A launch that touches at least this many bytes streams past the last-level cache.
constexpr size_t kStreamingBytes = 128u << 20;

// V consecutive 32-bit values, aligned for the widest single access (128 bits).
template<int V>
struct __attribute__((aligned(V >= 4 ? 16 : V * 4))) Pack {
    float v[V];
};

template<int V>
struct __attribute__((aligned(V >= 4 ? 16 : V * 4))) IPack {
    int v[V];
};

template<int V, bool NT = false>
__device__ __forceinline__ Pack<V> ld(const float* p, size_t e)
{
    Pack<V> r;
    if constexpr (!NT) {
        r = *reinterpret_cast<const Pack<V>*>(p + e);
    } else if constexpr (V == 1) {
        r.v[0] = __builtin_nontemporal_load(p + e);
    } else if constexpr (V == 2) {
        const f32x2 t = __builtin_nontemporal_load(reinterpret_cast<const f32x2*>(p + e));
        r.v[0] = t.x; r.v[1] = t.y;
    } else {
        static_assert(V % 4 == 0, "vector width");
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
            const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + e) + q);
            r.v[4 * q] = t.x; r.v[4 * q + 1] = t.y; r.v[4 * q + 2] = t.z; r.v[4 * q + 3] = t.w;
        }
    }
    return r;
}

template<int V, bool NT = false>
__device__ __forceinline__ void st(float* p, size_t e, const Pack<V>& v)
{
    if constexpr (!NT) {
        *reinterpret_cast<Pack<V>*>(p + e) = v;
    } else if constexpr (V == 1) {
        __builtin_nontemporal_store(v.v[0], p + e);
    } else if constexpr (V == 2) {
        f32x2 t; t.x = v.v[0]; t.y = v.v[1];
        __builtin_nontemporal_store(t, reinterpret_cast<f32x2*>(p + e));
    } else {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
            f32x4 t; t.x = v.v[4 * q]; t.y = v.v[4 * q + 1]; t.z = v.v[4 * q + 2]; t.w = v.v[4 * q + 3];
            __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(p + e) + q);
        }
    }
}

template<int V, bool NT = false>
__device__ __forceinline__ IPack<V> ldi(const int* p, size_t e)
{
    const Pack<V> t = ld<V, NT>(reinterpret_cast<const float*>(p), e);
    IPack<V> r;
#pragma unroll
    for (int k = 0; k < V; ++k) r.v[k] = __float_as_int(t.v[k]);
    return r;
}

template<int V, bool NT = false>
__device__ __forceinline__ void sti(int* p, size_t e, const IPack<V>& v)
{
    Pack<V> t;
#pragma unroll
    for (int k = 0; k < V; ++k) t.v[k] = __int_as_float(v.v[k]);
    st<V, NT>(reinterpret_cast<float*>(p), e, t);
}

// n_vec elements [0, n_vec) are processed V at a time (n_vec % V == 0), one vector per lane.
template<int V, bool NT, typename Op>
__global__ __launch_bounds__(kBlock) void stream_kernel(size_t n_vec, Op op)
{
    const size_t e = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * V;
    if (e < n_vec) {
        typename Op::template Regs<V> r;
        op.template load<V, NT>(e, r);
        op.template finish<V, NT>(e, r);
    }
}

// The same with two vectors per lane, a workgroup's width apart, all loads before the first store.  For
// the one operation here that reads four streams and writes four (the Adam update): measured with a
// plain kernel of that mix, 5.3 TB/s with one vector per lane and 5.75 with two; every other mix on
// this path (1 + 1 up to 3 + 2 streams) is as fast or faster with one.  Lanes past the end load element
// 0 (no branch between the loads) and store nothing.
template<bool NT, typename Op>
__global__ __launch_bounds__(kBlock) void stream_pairs_kernel(size_t n_vec, Op op)
{
    const size_t e0 = (static_cast<size_t>(blockIdx.x) * 2 * kBlock + threadIdx.x) * 4;
    const size_t e1 = e0 + static_cast<size_t>(kBlock) * 4;
    const bool in0 = e0 < n_vec, in1 = e1 < n_vec;
    typename Op::template Regs<4> r0, r1;
    op.template load<4, NT>(in0 ? e0 : 0, r0);
    op.template load<4, NT>(in1 ? e1 : 0, r1);
    if (in0) op.template finish<4, NT>(e0, r0);
    if (in1) op.template finish<4, NT>(e1, r1);
}

// Elements [begin, n) one at a time (the tail of the 128-bit path).
template<typename Op>
__global__ __launch_bounds__(kWave) void stream_tail_kernel(size_t begin, size_t n, Op op)
{
    const size_t e = begin + threadIdx.x;
    if (e < n) {
        typename Op::template Regs<1> r;
        op.template load<1, false>(e, r);
        op.template finish<1, false>(e, r);
    }
}

// ---------------------------------------------------------------- group sums of a written tensor
// Layer::backward opens with the L2 norm and the largest magnitude of the layer's delta
// (include/Layer.h:385-397, 479-499).  A flat kernel that is the last to write that delta can leave
// them behind per group of 256 values -- one wave's vectors -- and spare the tensor a read: the sum
// of squares of a group is wave_sum_by_rows over the lanes of ((x0^2 + x1^2) + x2^2) + x3^2, the order
// in which the norm pass itself adds, so the norm comes out the same to the bit either way.
__device__ __forceinline__ float square_sum(const Pack<4>& v)
{
    return ((v.v[0] * v.v[0] + v.v[1] * v.v[1]) + v.v[2] * v.v[2]) + v.v[3] * v.v[3];
}

__device__ __forceinline__ float peak_of(const Pack<4>& v)      // NaN-free unless all four are NaN
{
    return fmaxf(fmaxf(fabsf(v.v[0]), fabsf(v.v[1])), fmaxf(fabsf(v.v[2]), fabsf(v.v[3])));
}

constexpr int kGroupValues = kWave * 4;

// The op also supplies
//     template<int V, bool NT> __device__ Pack<V> finish_value(size_t e, const Regs<V>&) const;
// which does what finish does and returns the values it left in the tensor the groups describe.
// groups[g] = (sum of squares, largest magnitude) of values [256 g, 256 g + 256); n_vec % 4 == 0.
template<bool NT, typename Op>
__global__ __launch_bounds__(kBlock) void stream_groups_kernel(size_t n_vec, Op op, float2* groups)
{
    const size_t e = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    float a = 0.0f, peak = 0.0f;
    if (e < n_vec) {
        typename Op::template Regs<4> r;
        op.template load<4, NT>(e, r);
        const Pack<4> v = op.template finish_value<4, NT>(e, r);
        a = square_sum(v);
        peak = peak_of(v);
    }
    a = wave_sum_by_rows(a);
    peak = wave_max_by_rows(peak);
    const size_t first = (static_cast<size_t>(blockIdx.x) * kBlock + (threadIdx.x & ~(kWave - 1))) * 4;
    if ((threadIdx.x & (kWave - 1)) == 0 && first < n_vec) groups[first / kGroupValues] = make_float2(a, peak);
}

// Launches op over n elements (n % 4 == 0, every pointer 16-byte aligned) and leaves the group sums.
template<typename Op>
int launch_stream_groups(const char* name, size_t n, int bytes_per_elem, const Op& op, float2* groups,
                         hipStream_t stream)
{
    if (n == 0) return PXH_OK;
    const bool nt = n * static_cast<size_t>(bytes_per_elem) >= kStreamingBytes;
    const dim3 grid(grid_for(n, static_cast<size_t>(kBlock) * 4));
    if (nt) hipLaunchKernelGGL((stream_groups_kernel<true, Op>), grid, dim3(kBlock), 0, stream, n, op, groups);
    else hipLaunchKernelGGL((stream_groups_kernel<false, Op>), grid, dim3(kBlock), 0, stream, n, op, groups);
    return check_launch(name);
}

// Launches op over n elements.  `vector_ok`: every pointer the op touches is 16-byte aligned.
// `bytes_per_elem`: bytes the op moves per element, which picks the non-temporal variant from
// `streaming_from` bytes per launch on.
// `pairs`: two vectors per lane once the launch streams past the cache (stream_pairs_kernel).
template<typename Op>
int launch_stream(const char* name, size_t n, bool vector_ok, int bytes_per_elem, const Op& op, hipStream_t stream,
                  size_t streaming_from = kStreamingBytes, bool pairs = false)
{
    if (n == 0) return PXH_OK;
    const bool nt = n * static_cast<size_t>(bytes_per_elem) >= streaming_from;
    if (vector_ok) {
        const size_t n4 = n & ~static_cast<size_t>(3);
        if (n4) {
            const dim3 grid(grid_for(n4, static_cast<size_t>(kBlock) * 4));
            if (nt && pairs)
                hipLaunchKernelGGL((stream_pairs_kernel<true, Op>), dim3(grid_for(n4, static_cast<size_t>(kBlock) * 8)),
                                   dim3(kBlock), 0, stream, n4, op);
            else if (nt) hipLaunchKernelGGL((stream_kernel<4, true, Op>), grid, dim3(kBlock), 0, stream, n4, op);
            else hipLaunchKernelGGL((stream_kernel<4, false, Op>), grid, dim3(kBlock), 0, stream, n4, op);
        }
        if (n4 < n) {
            hipLaunchKernelGGL((stream_tail_kernel<Op>), dim3(1), dim3(kWave), 0, stream, n4, n, op);
        }
    } else {
        hipLaunchKernelGGL((stream_kernel<1, false, Op>), dim3(grid_for(n, kBlock)), dim3(kBlock), 0, stream, n, op);
    }
    return check_launch(name);
}

}  // namespace pxh
