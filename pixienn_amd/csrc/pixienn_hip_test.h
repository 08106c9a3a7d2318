/*
 * Test hooks of libpixienn_hip.so.  Exported so that the test-suite can reach them through the
 * shared library, but not part of the C ABI in include/pixienn_hip.h: nothing here is installed,
 * no host should call these, and none of them has a counterpart in the reference.
 */
#ifndef PIXIENN_HIP_TEST_H
#define PIXIENN_HIP_TEST_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* n / d through the multiply-high division the index maps use (n < 2^31, d >= 1).  Host only. */
unsigned pxh_debug_fastdiv(unsigned n, unsigned d);

/* Number (1..6) of whole-array sweeps of pxh_nms's duplicate step before the per-image loop finishes
 * what they left; returns the previous value.  Results do not depend on it.  A call of pxh_nms reads
 * it once, when it starts. */
int pxh_debug_nms_sweeps(int sweeps);

/* Address of the current device's library workspace after making it hold at least `bytes`
 * (NULL when that fails): lets a test see that a block handed out earlier stays where it was. */
void* pxh_debug_library_workspace(size_t bytes);

/* Forces the shape of the YOLO training pass for the calls that follow: its form (1 = one launch,
 * 2 = two launches) and, for the one-launch form, lanes per slot (1, 2 or 4) and the number of
 * persistent head workgroups; 0 = let the library choose.  Results do not depend on any of them beyond
 * the order of a few fp32 additions.  Returns 0. */
int pxh_debug_yolo_tuning(int form, int lanes_per_slot, int head_workers);

/* A kernel with no arithmetic to speak of that reads `reads` and writes `writes` streams of n floats each
 * (1 <= reads, writes <= 4; every pointer 16-byte aligned; n % 4 == 0), launched as the library launches
 * its streaming kernels: what that mix of reads and writes costs on the device whatever is computed.
 * in / out: host arrays of device pointers. */
int pxh_debug_stream_mix(int reads, int writes, size_t n, const float* const* in, float* const* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif
