// Host-side helpers of the C ABI: error reporting, argument validation, launch geometry.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/hyc_abi.h"
#include "row_codec.hpp"

namespace hyc {

char* error_buffer();   // thread-local, 512 bytes (abi.hip)

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

inline int ilog2(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return l;
}

// Geometry of one row under the chunk mapping.
struct RowGeom {
  int bits, nseg, cps, threads, iters;
  int64_t H, seg;
};

// H must make every segment a whole number of 8-channel chunks: H % (64/bits) == 0.
inline int row_geom(int64_t H, int bits, RowGeom* g) {
  if (!(bits == 1 || bits == 2 || bits == 4 || bits == 8)) return fail(HYC_ENOTSUP, "bits=%d: only 1, 2, 4, 8", bits);
  if (H <= 0 || H > 65536) return fail(HYC_EINVAL, "H=%lld out of range (1..65536)", (long long)H);
  const int per = 64 / bits;
  if (H % per != 0) return fail(HYC_ENOTSUP, "H=%lld must be a multiple of %d for %d-bit codes", (long long)H, per, bits);
  g->bits = bits;
  g->nseg = 8 / bits;
  g->H = H;
  g->seg = H / g->nseg;
  g->cps = (int)(g->seg / 8);
  int iters = 1;
  while ((g->cps + iters - 1) / iters > 1024) ++iters;
  int t = (g->cps + iters - 1) / iters;
  t = ((t + 63) / 64) * 64;
  g->threads = t;
  g->iters = (g->cps + t - 1) / t;
  return HYC_OK;
}

// Channel-mode checks: the group must be 8*2^n channels (n = 2..6) and divide a segment.
inline int chan_geom(const RowGeom& g, int group, int* lpg) {
  if (group < 32 || group > 512 || (group & (group - 1)) != 0)
    return fail(HYC_ENOTSUP, "group=%d: supported group sizes are 32, 64, 128, 256, 512", group);
  if (g.seg % group != 0)
    return fail(HYC_ENOTSUP, "group=%d must divide the segment length H*bits/8=%lld", group, (long long)g.seg);
  *lpg = group / 8;
  return HYC_OK;
}

// The HIP runtime keeps the last error of the thread until it is read; other code in the process (the
// framework that owns the streams) may have left one behind.  Entry points call this before they launch so
// that check_launch() reports only their own failure.
inline void drop_stale_error() { (void)hipGetLastError(); }
inline hipStream_t begin_launch(void* stream) {
  drop_stale_error();
  return static_cast<hipStream_t>(stream);
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HYC_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return HYC_OK;
}

inline float round_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  u &= 0xFFFF0000u;
  memcpy(&f, &u, 4);
  return f;
}

// Fill the device-side views of a descriptor.  Validates what the given mode needs.
int make_chan_args(const hyc_desc* d, const RowGeom& g, ChanArgs* a, int* lpg);
int make_thr_args(const hyc_desc* d, const RowGeom& g, ThrArgs* a, bool* perchan);

}  // namespace hyc
