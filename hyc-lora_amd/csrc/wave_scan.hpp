// Ordered compaction inside one wave (gfx950, wave64): a prefix sum over the lanes through DPP row shifts and row
// broadcasts (six data-parallel adds, no LDS traffic), and a staging row in LDS from which a wave stores the entries
// it kept as contiguous runs instead of one scattered store per entry.
#pragma once
#include <stdint.h>

namespace hyc {

// inclusive prefix sum of `v` over the 64 lanes: lane L returns v[0] + ... + v[L].  Every lane must take part.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  // inside each row of 16 lanes (lanes without a source add the 0 of `old`) ...
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
  // ... then the last lane of a row to the next row (rows 1 and 3), and lane 31 to rows 2 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31
  return v;
}

// The kept entries (column, bf16 bits) of one row, in column order.  The first STAGE_CAP of them wait in the wave's
// staging row (one 32-bit word each: column in the low half, value in the high half; columns stay below 65 536) and
// leave through flush(); entries beyond that go to memory one by one.  `limit` = the room the row has in cols / vals
// (row_ptr[row + 1] - row_ptr[row]): it equals the row's count unless the caller's offsets were cut off at the capacity
// of its buffers, in which case the entries past it are dropped (the caller learns of it from the total it asked for).
constexpr int STAGE_CAP = 1024;

__device__ __forceinline__ void stage_entry(uint32_t* stage, int pos, int limit, int col, uint16_t bits, int32_t* cols_row,
                                            uint16_t* vals_row) {
  if (pos < STAGE_CAP) {
    stage[pos] = (uint32_t)col | ((uint32_t)bits << 16);
  } else if (pos < limit) {
    cols_row[pos] = col;
    vals_row[pos] = bits;
  }
}

// `count` = entries of the row; every lane of the wave calls this after the last stage_entry() of the row
__device__ __forceinline__ void stage_flush(const uint32_t* stage, int count, int limit, int32_t* cols_row, uint16_t* vals_row) {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   // the other lanes' staging writes before these reads
  __builtin_amdgcn_wave_barrier();
  const int lane = threadIdx.x & 63;
  count = count < limit ? count : limit;
  const int n = count < STAGE_CAP ? count : STAGE_CAP;
  for (int e = lane; e < n; e += 64) {
    const uint32_t w = stage[e];
    cols_row[e] = (int32_t)(w & 0xFFFFu);
    vals_row[e] = (uint16_t)(w >> 16);
  }
}

}  // namespace hyc
