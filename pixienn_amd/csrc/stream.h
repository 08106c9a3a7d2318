// Flat streaming skeleton: one workgroup covers kChunk consecutive elements, each lane issues
// kUnroll 128-bit loads per stream before it computes or stores anything, so a wavefront keeps
// kUnroll KiB per stream in flight.  An operation supplies
//     template<int V> struct Regs;                       // what it keeps between load and finish
//     template<int V> __device__ void load(size_t e, Regs<V>&) const;    // e = first element
//     template<int V> __device__ void finish(size_t e, const Regs<V>&) const;
// V is 4 for the 128-bit path and 1 for the scalar path (unaligned pointers and the n % 4 tail).
#pragma once

#include "common.h"

namespace pxh {

// V consecutive 32-bit values, aligned for the widest single load (128 bits).
template<int V>
struct __attribute__((aligned(V >= 4 ? 16 : V * 4))) Pack {
    float v[V];
};

template<int V>
struct __attribute__((aligned(V >= 4 ? 16 : V * 4))) IPack {
    int v[V];
};

template<int V>
__device__ __forceinline__ Pack<V> ld(const float* p, size_t e)
{
    return *reinterpret_cast<const Pack<V>*>(p + e);
}

template<int V>
__device__ __forceinline__ void st(float* p, size_t e, const Pack<V>& v)
{
    *reinterpret_cast<Pack<V>*>(p + e) = v;
}

template<int V>
__device__ __forceinline__ IPack<V> ldi(const int* p, size_t e)
{
    return *reinterpret_cast<const IPack<V>*>(p + e);
}

template<int V>
__device__ __forceinline__ void sti(int* p, size_t e, const IPack<V>& v)
{
    *reinterpret_cast<IPack<V>*>(p + e) = v;
}

// n_vec elements [0, n_vec) are processed V at a time (n_vec % V == 0).
template<int V, typename Op>
__global__ __launch_bounds__(kBlock) void stream_kernel(size_t n_vec, Op op)
{
    const size_t base = (static_cast<size_t>(blockIdx.x) * kBlock * kUnroll + threadIdx.x) * V;
    typename Op::template Regs<V> r[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const size_t e = base + static_cast<size_t>(u) * kBlock * V;
        if (e < n_vec) op.template load<V>(e, r[u]);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const size_t e = base + static_cast<size_t>(u) * kBlock * V;
        if (e < n_vec) op.template finish<V>(e, r[u]);
    }
}

// Elements [begin, n) one at a time (the tail of the 128-bit path).
template<typename Op>
__global__ __launch_bounds__(kWave) void stream_tail_kernel(size_t begin, size_t n, Op op)
{
    const size_t e = begin + threadIdx.x;
    if (e < n) {
        typename Op::template Regs<1> r;
        op.template load<1>(e, r);
        op.template finish<1>(e, r);
    }
}

// Launches op over n elements; `vector_ok` says every pointer the op touches is 16-byte aligned.
template<typename Op>
int launch_stream(const char* name, size_t n, bool vector_ok, const Op& op, hipStream_t stream)
{
    if (n == 0) return PXH_OK;
    if (vector_ok) {
        const size_t n4 = n & ~static_cast<size_t>(3);
        if (n4) {
            const size_t per_block = static_cast<size_t>(kBlock) * kUnroll * 4;
            hipLaunchKernelGGL((stream_kernel<4, Op>), dim3(grid_for(n4, per_block)), dim3(kBlock), 0, stream,
                               n4, op);
        }
        if (n4 < n) {
            hipLaunchKernelGGL((stream_tail_kernel<Op>), dim3(1), dim3(kWave), 0, stream, n4, n, op);
        }
    } else {
        const size_t per_block = static_cast<size_t>(kBlock) * kUnroll;
        hipLaunchKernelGGL((stream_kernel<1, Op>), dim3(grid_for(n, per_block)), dim3(kBlock), 0, stream, n, op);
    }
    return check_launch(name);
}

// ---------------------------------------------------------------- NCHW plane lookup
// Maps a flat element index to its channel with one multiply-high division.
struct PlaneMap {
    FastDiv by_spatial;
    FastDiv by_channels;
    PlaneMap() {}
    PlaneMap(int channels, int spatial)
        : by_spatial(static_cast<uint32_t>(spatial)), by_channels(static_cast<uint32_t>(channels)) {}
    // element index -> (channel, offset inside the plane)
    __device__ __forceinline__ void locate(size_t e, uint32_t& channel, uint32_t& offset) const
    {
        uint32_t plane, q;
        by_spatial.divmod(static_cast<uint32_t>(e), plane, offset);
        by_channels.divmod(plane, q, channel);
    }
    __device__ __forceinline__ uint32_t next_channel(uint32_t channel) const
    {
        return channel + 1 == by_channels.d ? 0 : channel + 1;
    }
};

}  // namespace pxh
