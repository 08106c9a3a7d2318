// Max-pool (values + int32 argmax) and nearest upsample, forward and backward, for gfx950.
// Index and copy work is bit-exact against the CPU layers; accumulation follows their order.
#include "stream.h"

#include <cfloat>

namespace pxh {
namespace {

struct PoolGeom {
    int ih, iw, oh, ow, kernel, stride, origin;   // origin = -padding / 2
};

// ------------------------------------------------------------------ max-pool, any geometry
// One output per lane.  Taps in row-major order; the first in-bounds tap is taken, later taps
// only when strictly greater (include/MaxPoolLayer.h:106-127 of the reference).
__global__ __launch_bounds__(kBlock) void maxpool_fwd_generic_kernel(const float* in, float* out, int* indexes,
                                                                     uint32_t total, PoolGeom g, FastDiv by_ow,
                                                                     FastDiv by_oh)
{
    const uint32_t o = blockIdx.x * kBlock + threadIdx.x;
    if (o >= total) return;
    uint32_t rows, ox, plane, oy;
    by_ow.divmod(o, rows, ox);
    by_oh.divmod(rows, plane, oy);
    float best = -FLT_MAX;
    int best_at = -1;
    for (int ky = 0; ky < g.kernel; ++ky) {
        const int y = g.origin + static_cast<int>(oy) * g.stride + ky;
        if (y < 0 || y >= g.ih) continue;
        for (int kx = 0; kx < g.kernel; ++kx) {
            const int x = g.origin + static_cast<int>(ox) * g.stride + kx;
            if (x < 0 || x >= g.iw) continue;
            const int at = x + g.iw * (y + g.ih * static_cast<int>(plane));
            const float v = in[at];
            if (best_at < 0 || v > best) {
                best_at = at;
                best = v;
            }
        }
    }
    out[o] = best;
    indexes[o] = best_at;
}

// 2x2 / stride 2 windows that all lie inside the input: VX outputs per lane from two
// (2*VX)-wide row loads, stored as VX-wide value and index vectors.
template<int VX, bool NT>
__global__ __launch_bounds__(kBlock) void maxpool_fwd_2x2_kernel(const float* in, float* out, int* indexes,
                                                                 uint32_t units, int iw, int ow, FastDiv by_owv,
                                                                 FastDiv by_oh)
{
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= units) return;
    uint32_t rows, oxv, plane, oy;
    by_owv.divmod(t, rows, oxv);
    by_oh.divmod(rows, plane, oy);
    const uint32_t ih = by_oh.d * 2;
    const uint32_t ox = oxv * VX;
    const uint32_t in0 = (plane * ih + 2 * oy) * iw + 2 * ox;   // < 2^31 checked by the host
    const Pack<2 * VX> r0 = ld<2 * VX, NT>(in, in0);
    const Pack<2 * VX> r1 = ld<2 * VX, NT>(in, in0 + iw);
    Pack<VX> v;
    IPack<VX> ix;
#pragma unroll
    for (int k = 0; k < VX; ++k) {
        float best = r0.v[2 * k];
        int at = in0 + 2 * k;
        if (r0.v[2 * k + 1] > best) { best = r0.v[2 * k + 1]; at = in0 + 2 * k + 1; }
        if (r1.v[2 * k] > best) { best = r1.v[2 * k]; at = in0 + iw + 2 * k; }
        if (r1.v[2 * k + 1] > best) { best = r1.v[2 * k + 1]; at = in0 + iw + 2 * k + 1; }
        v.v[k] = best;
        ix.v[k] = at;
    }
    const uint32_t o = (plane * by_oh.d + oy) * ow + ox;
    st<VX, NT>(out, o, v);
    sti<VX, NT>(indexes, o, ix);
}

// The same for an even output width (input rows of a multiple of 4 floats) and a multiple of 4
// outputs in all, with one 128-bit access per lane and stream: a lane takes 2 consecutive
// outputs of the flat output tensor (they share a row), i.e. 4 floats of each of two input rows;
// the lanes of a pair then swap halves so that the even lane stores the pair's 4 values and the
// odd lane its 4 indexes.  Every address is 16-byte aligned: rows start at multiples of 4 floats.
template<bool NT>
__global__ __launch_bounds__(kBlock) void maxpool_fwd_2x2_pair_kernel(const float* in, float* out, int* indexes,
                                                                      uint32_t lanes, int iw, int ow, FastDiv by_owh,
                                                                      FastDiv by_oh)
{
    // the grid is a whole number of waves and `lanes` is even: a pair is never split by the guard
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    const bool live = t < lanes;
    const uint32_t u = live ? t : 0;
    const uint32_t half = u & 1;
    uint32_t rows, oxh, plane, oy;
    by_owh.divmod(u, rows, oxh);
    by_oh.divmod(rows, plane, oy);
    const uint32_t ih = by_oh.d * 2;
    const uint32_t ox = oxh * 2;
    const uint32_t in0 = (plane * ih + 2 * oy) * iw + 2 * ox;   // < 2^31 checked by the host
    const Pack<4> r0 = ld<4, NT>(in, in0);
    const Pack<4> r1 = ld<4, NT>(in, in0 + iw);
    float v[2];
    int ix[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        float best = r0.v[2 * k];
        int at = in0 + 2 * k;
        if (r0.v[2 * k + 1] > best) { best = r0.v[2 * k + 1]; at = in0 + 2 * k + 1; }
        if (r1.v[2 * k] > best) { best = r1.v[2 * k]; at = in0 + iw + 2 * k; }
        if (r1.v[2 * k + 1] > best) { best = r1.v[2 * k + 1]; at = in0 + iw + 2 * k + 1; }
        v[k] = best;
        ix[k] = at;
    }
    // even lane: gives its indexes, takes the partner's values; odd lane the other way round
    const float pv0 = __shfl_xor(v[0], 1, kWave), pv1 = __shfl_xor(v[1], 1, kWave);
    const int pi0 = __shfl_xor(ix[0], 1, kWave), pi1 = __shfl_xor(ix[1], 1, kWave);
    if (!live) return;
    const uint32_t o = (u >> 1) * 4;       // the pair's 4 flat outputs
    if (half == 0) {
        const Pack<4> w{ { v[0], v[1], pv0, pv1 } };
        st<4, NT>(out, o, w);
    } else {
        const IPack<4> w{ { pi0, pi1, ix[0], ix[1] } };
        sti<4, NT>(indexes, o, w);
    }
}

// Backward, any geometry: one input cell per lane gathers, in ascending output order, the
// deltas of the windows whose recorded argmax is this cell.  Ascending output order is the
// order in which the sequential CPU loop reaches this cell (include/MaxPoolLayer.h:150-156).
__global__ __launch_bounds__(kBlock) void maxpool_bwd_generic_kernel(const float* delta, const int* indexes,
                                                                     float* grad, uint32_t total, PoolGeom g,
                                                                     FastDiv by_iw, FastDiv by_ih)
{
    const uint32_t cell = blockIdx.x * kBlock + threadIdx.x;
    if (cell >= total) return;
    uint32_t rows, x, plane, y;
    by_iw.divmod(cell, rows, x);
    by_ih.divmod(rows, plane, y);
    // windows with origin + o*stride <= p <= origin + o*stride + kernel - 1
    const int py = static_cast<int>(y) - g.origin, px = static_cast<int>(x) - g.origin;
    int oy0 = py - g.kernel + 1;
    oy0 = oy0 <= 0 ? 0 : (oy0 + g.stride - 1) / g.stride;
    int ox0 = px - g.kernel + 1;
    ox0 = ox0 <= 0 ? 0 : (ox0 + g.stride - 1) / g.stride;
    const int oy1 = min(g.oh - 1, py >= 0 ? py / g.stride : -1);
    const int ox1 = min(g.ow - 1, px >= 0 ? px / g.stride : -1);
    float acc = grad[cell];
    bool touched = false;
    for (int oy = oy0; oy <= oy1; ++oy)
        for (int ox = ox0; ox <= ox1; ++ox) {
            const int o = ox + g.ow * (oy + g.oh * static_cast<int>(plane));
            if (indexes[o] == static_cast<int>(cell)) {
                acc += delta[o];
                touched = true;
            }
        }
    if (touched) grad[cell] = acc;
}

// Backward for the 2x2 / stride 2 in-bounds case: one window per output, VX windows per lane,
// the two grad rows are updated as full vectors so the read-modify-write stays coalesced.
template<int VX, bool NT>
__global__ __launch_bounds__(kBlock) void maxpool_bwd_2x2_kernel(const float* delta, const int* indexes, float* grad,
                                                                 uint32_t units, int iw, int ow, FastDiv by_owv,
                                                                 FastDiv by_oh)
{
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= units) return;
    uint32_t rows, oxv, plane, oy;
    by_owv.divmod(t, rows, oxv);
    by_oh.divmod(rows, plane, oy);
    const uint32_t ih = by_oh.d * 2;
    const uint32_t ox = oxv * VX;
    const uint32_t in0 = (plane * ih + 2 * oy) * iw + 2 * ox;
    const uint32_t o = (plane * by_oh.d + oy) * ow + ox;
    const Pack<VX> d = ld<VX, NT>(delta, o);
    const IPack<VX> ix = ldi<VX, NT>(indexes, o);
    Pack<2 * VX> g0 = ld<2 * VX, NT>(grad, in0);
    Pack<2 * VX> g1 = ld<2 * VX, NT>(grad, in0 + iw);
#pragma unroll
    for (int k = 0; k < VX; ++k) {
        const int at = ix.v[k];
        const int base = static_cast<int>(in0) + 2 * k;
        if (at == base) g0.v[2 * k] += d.v[k];
        else if (at == base + 1) g0.v[2 * k + 1] += d.v[k];
        else if (at == base + iw) g1.v[2 * k] += d.v[k];
        else if (at == base + iw + 1) g1.v[2 * k + 1] += d.v[k];
    }
    st<2 * VX, NT>(grad, in0, g0);
    st<2 * VX, NT>(grad, in0 + iw, g1);
}

// The pair form of the backward pass: the even lane reads the pair's 4 deltas, the odd lane its
// 4 indexes, they swap halves, and every lane updates 4 floats of each of the two grad rows.
template<bool NT>
__global__ __launch_bounds__(kBlock) void maxpool_bwd_2x2_pair_kernel(const float* delta, const int* indexes,
                                                                      float* grad, uint32_t lanes, int iw, int ow,
                                                                      FastDiv by_owh, FastDiv by_oh)
{
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    const bool live = t < lanes;
    const uint32_t u = live ? t : 0;
    const uint32_t half = u & 1;
    uint32_t rows, oxh, plane, oy;
    by_owh.divmod(u, rows, oxh);
    by_oh.divmod(rows, plane, oy);
    const uint32_t ih = by_oh.d * 2;
    const uint32_t ox = oxh * 2;
    const uint32_t in0 = (plane * ih + 2 * oy) * iw + 2 * ox;
    const uint32_t o = (u >> 1) * 4;
    // one 128-bit load per lane: deltas (even) or indexes (odd), as raw bits
    const Pack<4> mine = half == 0 ? ld<4, NT>(delta, o) : ld<4, NT>(reinterpret_cast<const float*>(indexes), o);
    Pack<4> theirs;
#pragma unroll
    for (int k = 0; k < 4; ++k) theirs.v[k] = __shfl_xor(mine.v[k], 1, kWave);
    // this lane's two windows are outputs 2*half, 2*half + 1 of the pair
    float d[2];
    int ix[2];
    if (half == 0) {
        d[0] = mine.v[0]; d[1] = mine.v[1];
        ix[0] = __float_as_int(theirs.v[0]); ix[1] = __float_as_int(theirs.v[1]);
    } else {
        d[0] = theirs.v[2]; d[1] = theirs.v[3];
        ix[0] = __float_as_int(mine.v[2]); ix[1] = __float_as_int(mine.v[3]);
    }
    if (!live) return;
    Pack<4> g0 = ld<4, NT>(grad, in0);
    Pack<4> g1 = ld<4, NT>(grad, in0 + iw);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int at = ix[k];
        const int base = static_cast<int>(in0) + 2 * k;
        if (at == base) g0.v[2 * k] += d[k];
        else if (at == base + 1) g0.v[2 * k + 1] += d[k];
        else if (at == base + iw) g1.v[2 * k] += d[k];
        else if (at == base + iw + 1) g1.v[2 * k + 1] += d[k];
    }
    st<4, NT>(grad, in0, g0);
    st<4, NT>(grad, in0 + iw, g1);
}

__global__ __launch_bounds__(kBlock) void maxpool_bwd_scatter_kernel(const float* delta, const int* indexes,
                                                                     float* grad, int size)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= size) return;
    const int at = indexes[i];
    if (at >= 0) atomicAdd(grad + at, delta[i]);
}

// ------------------------------------------------------------------ upsample
// The large tensor may be a channel slice of a wider one (a concatenation buffer): image n then
// starts `extra` elements later than in a dense tensor, for every image before it.
struct ImageGap {
    FastDiv by_channels;
    uint32_t extra;     // image stride of the large tensor minus channels * its plane size
    __device__ uint32_t of_plane(uint32_t plane) const { return extra ? by_channels.div(plane) * extra : 0u; }
};

// stride 2: VX inputs per lane; forward writes the 2 x (2*VX) block, backward folds it into the
// input cell as (((acc + s*o00) + s*o01) + s*o10) + s*o11, the raster order of the CPU loop.
template<int VX, bool FORWARD>
__global__ __launch_bounds__(kBlock) void upsample2_kernel(const float* in, float* acc, float* out, uint32_t units,
                                                           int w, float scale, FastDiv by_wv, FastDiv by_h,
                                                           ImageGap gap)
{
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= units) return;
    uint32_t rows, xv, plane, y;
    by_wv.divmod(t, rows, xv);
    by_h.divmod(rows, plane, y);
    const uint32_t x = xv * VX;
    const uint32_t ii = rows * w + x;                                   // rows = plane*h + y
    const uint32_t ow = 2 * w;
    const uint32_t oi = (2 * rows) * ow + 2 * x + gap.of_plane(plane);  // (plane*2h + 2y)*2w + 2x
    if constexpr (FORWARD) {
        const Pack<VX> v = ld<VX>(in, ii);
        Pack<2 * VX> o;
#pragma unroll
        for (int k = 0; k < VX; ++k) {
            const float s = scale * v.v[k];
            o.v[2 * k] = s;
            o.v[2 * k + 1] = s;
        }
        st<2 * VX>(out, oi, o);
        st<2 * VX>(out, oi + ow, o);
    } else {
        Pack<VX> a = ld<VX>(acc, ii);
        const Pack<2 * VX> r0 = ld<2 * VX>(out, oi);
        const Pack<2 * VX> r1 = ld<2 * VX>(out, oi + ow);
#pragma unroll
        for (int k = 0; k < VX; ++k) {
            float g = a.v[k];
            float p = scale * r0.v[2 * k];
            g = g + p;
            p = scale * r0.v[2 * k + 1];
            g = g + p;
            p = scale * r1.v[2 * k];
            g = g + p;
            p = scale * r1.v[2 * k + 1];
            g = g + p;
            a.v[k] = g;
        }
        st<VX>(acc, ii, a);
    }
}

// any stride: one input cell per lane
template<bool FORWARD>
__global__ __launch_bounds__(kBlock) void upsample_generic_kernel(const float* in, float* acc, float* out,
                                                                  uint32_t total, int w, int stride, float scale,
                                                                  FastDiv by_w, FastDiv by_h, ImageGap gap)
{
    const uint32_t cell = blockIdx.x * kBlock + threadIdx.x;
    if (cell >= total) return;
    uint32_t rows, x, plane, y;
    by_w.divmod(cell, rows, x);
    by_h.divmod(rows, plane, y);
    const size_t ow = static_cast<size_t>(w) * stride;
    const size_t o0 = static_cast<size_t>(rows) * stride * ow + static_cast<size_t>(x) * stride + gap.of_plane(plane);
    if constexpr (FORWARD) {
        const float s = scale * in[cell];
        for (int dy = 0; dy < stride; ++dy)
            for (int dx = 0; dx < stride; ++dx) out[o0 + dy * ow + dx] = s;
    } else {
        float g = acc[cell];
        for (int dy = 0; dy < stride; ++dy)
            for (int dx = 0; dx < stride; ++dx) {
                const float p = scale * out[o0 + dy * ow + dx];
                g = g + p;
            }
        acc[cell] = g;
    }
}

int check_pool_args(const char* who, int batch, int channels, int ih, int iw, int oh, int ow, int kernel, int stride,
                    int padding)
{
    if (batch <= 0 || channels <= 0 || ih <= 0 || iw <= 0 || oh <= 0 || ow <= 0)
        return fail_invalid("%s: dimensions must be positive", who);
    if (kernel <= 0) return fail_invalid("%s: MaxPool kernel must be positive", who);
    if (stride <= 0) return fail_invalid("%s: MaxPool stride must be positive", who);
    if (padding < 0) return fail_invalid("%s: MaxPool padding cannot be negative", who);
    const unsigned long long in_total = 1ull * batch * channels * ih * iw;
    const unsigned long long out_total = 1ull * batch * channels * oh * ow;
    if (in_total >= (1ull << 31) || out_total >= (1ull << 31)) {
        // the index tensor is int32: larger inputs cannot be represented by the layer at all
        set_error("%s: tensors of 2^31 elements or more are not supported", who);
        return PXH_ERR_UNSUPPORTED;
    }
    return PXH_OK;
}

// all windows 2x2, stride 2, inside the input
bool is_2x2_inbounds(int ih, int iw, int oh, int ow, int kernel, int stride, int padding)
{
    return kernel == 2 && stride == 2 && padding <= 1 && ih % 2 == 0 && iw % 2 == 0 && oh == ih / 2 && ow == iw / 2;
}

}  // namespace
}  // namespace pxh

using namespace pxh;

extern "C" {

int pxh_maxpool_forward(const float* in, float* out, int* indexes, int batch, int channels, int ih, int iw, int oh,
                        int ow, int kernel, int stride, int padding, void* stream)
{
    if (!in || !out || !indexes) return fail_invalid("pxh_maxpool_forward: null pointer");
    int rc = check_pool_args("pxh_maxpool_forward", batch, channels, ih, iw, oh, ow, kernel, stride, padding);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const uint32_t planes = static_cast<uint32_t>(batch) * channels;
    const uint32_t total = planes * oh * ow;
    if (is_2x2_inbounds(ih, iw, oh, ow, kernel, stride, padding) && aligned16(in) && aligned16(out) &&
        aligned16(indexes)) {
        // 4 bytes in, 8 bytes out per input element / 4
        const bool nt = static_cast<size_t>(total) * 24 >= kStreamingBytes;
        // the pair form needs an even output width and whole output quads; it pays for wide rows
        if (iw % 8 == 0 && total % 4 == 0) {
            const uint32_t lanes = total / 2;
            const dim3 grid(grid_for(lanes, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_fwd_2x2_pair_kernel<true>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                       lanes, iw, ow, FastDiv(ow / 2), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_fwd_2x2_pair_kernel<false>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                    lanes, iw, ow, FastDiv(ow / 2), FastDiv(oh));
        } else if (iw % 4 == 0) {
            const uint32_t units = total / 2;
            const dim3 grid(grid_for(units, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_fwd_2x2_kernel<2, true>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                       units, iw, ow, FastDiv(ow / 2), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_fwd_2x2_kernel<2, false>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                    units, iw, ow, FastDiv(ow / 2), FastDiv(oh));
        } else {
            const dim3 grid(grid_for(total, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_fwd_2x2_kernel<1, true>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                       total, iw, ow, FastDiv(ow), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_fwd_2x2_kernel<1, false>), grid, dim3(kBlock), 0, s, in, out, indexes,
                                    total, iw, ow, FastDiv(ow), FastDiv(oh));
        }
        return check_launch("pxh_maxpool_forward");
    }
    const PoolGeom g{ ih, iw, oh, ow, kernel, stride, -padding / 2 };
    hipLaunchKernelGGL(maxpool_fwd_generic_kernel, dim3(grid_for(total, kBlock)), dim3(kBlock), 0, s, in, out, indexes,
                       total, g, FastDiv(ow), FastDiv(oh));
    return check_launch("pxh_maxpool_forward");
}

int pxh_maxpool_backward(const float* delta, const int* indexes, float* grad, int batch, int channels, int ih, int iw,
                         int oh, int ow, int kernel, int stride, int padding, void* stream)
{
    if (!delta || !indexes || !grad) return fail_invalid("pxh_maxpool_backward: null pointer");
    int rc = check_pool_args("pxh_maxpool_backward", batch, channels, ih, iw, oh, ow, kernel, stride, padding);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const uint32_t planes = static_cast<uint32_t>(batch) * channels;
    const uint32_t out_total = planes * oh * ow;
    if (is_2x2_inbounds(ih, iw, oh, ow, kernel, stride, padding) && aligned16(delta) && aligned16(indexes) &&
        aligned16(grad)) {
        // 8 bytes per output, 8 bytes per grad cell
        const bool nt = static_cast<size_t>(out_total) * 40 >= kStreamingBytes;
        if (iw % 8 == 0 && out_total % 4 == 0) {
            const uint32_t lanes = out_total / 2;
            const dim3 grid(grid_for(lanes, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_bwd_2x2_pair_kernel<true>), grid, dim3(kBlock), 0, s, delta, indexes,
                                       grad, lanes, iw, ow, FastDiv(ow / 2), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_bwd_2x2_pair_kernel<false>), grid, dim3(kBlock), 0, s, delta, indexes,
                                    grad, lanes, iw, ow, FastDiv(ow / 2), FastDiv(oh));
        } else if (iw % 4 == 0) {
            const uint32_t units = out_total / 2;
            const dim3 grid(grid_for(units, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_bwd_2x2_kernel<2, true>), grid, dim3(kBlock), 0, s, delta, indexes,
                                       grad, units, iw, ow, FastDiv(ow / 2), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_bwd_2x2_kernel<2, false>), grid, dim3(kBlock), 0, s, delta, indexes, grad,
                                    units, iw, ow, FastDiv(ow / 2), FastDiv(oh));
        } else {
            const dim3 grid(grid_for(out_total, kBlock));
            if (nt) hipLaunchKernelGGL((maxpool_bwd_2x2_kernel<1, true>), grid, dim3(kBlock), 0, s, delta, indexes,
                                       grad, out_total, iw, ow, FastDiv(ow), FastDiv(oh));
            else hipLaunchKernelGGL((maxpool_bwd_2x2_kernel<1, false>), grid, dim3(kBlock), 0, s, delta, indexes, grad,
                                    out_total, iw, ow, FastDiv(ow), FastDiv(oh));
        }
        return check_launch("pxh_maxpool_backward");
    }
    const PoolGeom g{ ih, iw, oh, ow, kernel, stride, -padding / 2 };
    const uint32_t in_total = planes * ih * iw;
    hipLaunchKernelGGL(maxpool_bwd_generic_kernel, dim3(grid_for(in_total, kBlock)), dim3(kBlock), 0, s, delta,
                       indexes, grad, in_total, g, FastDiv(iw), FastDiv(ih));
    return check_launch("pxh_maxpool_backward");
}

int pxh_maxpool_backward_scatter(const float* delta, const int* indexes, float* grad, int size, void* stream)
{
    if (size < 0 || ((!delta || !indexes || !grad) && size)) return fail_invalid("pxh_maxpool_backward_scatter: bad argument");
    if (size == 0) return PXH_OK;
    hipLaunchKernelGGL(maxpool_bwd_scatter_kernel, dim3(grid_for(size, kBlock)), dim3(kBlock), 0, as_stream(stream),
                       delta, indexes, grad, size);
    return check_launch("pxh_maxpool_backward_scatter");
}

int pxh_upsample_strided(const float* in, int w, int h, int c, int batch, int stride, int forward, float scale,
                         float* acc, float* out, long long out_image_stride, void* stream)
{
    if (w <= 0 || h <= 0 || c <= 0 || batch <= 0 || stride <= 0)
        return fail_invalid("pxh_upsample: dimensions and stride must be positive");
    if (!out || (forward && !in) || (!forward && !acc)) return fail_invalid("pxh_upsample: null pointer");
    const unsigned long long image = 1ull * c * h * w * stride * stride;
    if (out_image_stride < 0 || static_cast<unsigned long long>(out_image_stride) < image)
        return fail_invalid("pxh_upsample: image stride %lld is smaller than one upsampled image (%llu)",
                            out_image_stride, image);
    if (1ull * batch * static_cast<unsigned long long>(out_image_stride) >= (1ull << 31)) {
        set_error("pxh_upsample: tensors of 2^31 elements or more are not supported");
        return PXH_ERR_UNSUPPORTED;
    }
    hipStream_t s = as_stream(stream);
    const uint32_t total = static_cast<uint32_t>(batch) * c * h * w;
    const ImageGap gap{ FastDiv(c), static_cast<uint32_t>(static_cast<unsigned long long>(out_image_stride) - image) };
    const float* small = forward ? in : acc;
    if (stride == 2 && aligned16(small) && aligned16(out) && gap.extra % 4 == 0) {
        // VX inputs per lane; the input vector needs 4*VX-byte alignment of every row start
        const int vx = (w % 4 == 0) ? 4 : (w % 2 == 0 ? 2 : 1);
        const uint32_t units = total / vx;
        const dim3 grid(grid_for(units, kBlock));
#define PXH_UPSAMPLE2(VX, FWD)                                                                              \
        hipLaunchKernelGGL((upsample2_kernel<VX, FWD>), grid, dim3(kBlock), 0, s, in, acc, out, units, w, \
                           scale, FastDiv(w / VX), FastDiv(h), gap)
        if (forward) {
            if (vx == 4) PXH_UPSAMPLE2(4, true); else if (vx == 2) PXH_UPSAMPLE2(2, true); else PXH_UPSAMPLE2(1, true);
        } else {
            if (vx == 4) PXH_UPSAMPLE2(4, false); else if (vx == 2) PXH_UPSAMPLE2(2, false); else PXH_UPSAMPLE2(1, false);
        }
#undef PXH_UPSAMPLE2
        return check_launch("pxh_upsample");
    }
    const dim3 grid(grid_for(total, kBlock));
    if (forward) {
        hipLaunchKernelGGL((upsample_generic_kernel<true>), grid, dim3(kBlock), 0, s, in, acc, out, total, w, stride,
                           scale, FastDiv(w), FastDiv(h), gap);
    } else {
        hipLaunchKernelGGL((upsample_generic_kernel<false>), grid, dim3(kBlock), 0, s, in, acc, out, total, w, stride,
                           scale, FastDiv(w), FastDiv(h), gap);
    }
    return check_launch("pxh_upsample");
}

int pxh_upsample(const float* in, int w, int h, int c, int batch, int stride, int forward, float scale, float* acc,
                 float* out, void* stream)
{
    if (w <= 0 || h <= 0 || c <= 0 || batch <= 0 || stride <= 0)
        return fail_invalid("pxh_upsample: dimensions and stride must be positive");
    return pxh_upsample_strided(in, w, h, c, batch, stride, forward, scale, acc, out,
                                1ll * c * h * w * stride * stride, stream);
}

}
