// Row encoders / decoders: the per-iteration work of one thread on its NSEG chunks.
// Used by the standalone compress / decompress kernels and fused into the RMSNorm, activation and
// weight-gradient kernels.
#pragma once
#include "row_codec.hpp"

namespace hyc {

__device__ __forceinline__ uint16_t raw16(const uint4& r, int j) {
  const uint32_t w = (j < 2) ? r.x : (j < 4) ? r.y : (j < 6) ? r.z : r.w;
  return (uint16_t)((j & 1) ? (w >> 16) : (w & 0xFFFF));
}

// ------------------------------------------------------------------------------------------------
// channel mode
// ------------------------------------------------------------------------------------------------
// Encode the NSEG chunks `raw` (chunk index c of each segment) of one row.  Every lane of the wave must
// call this (inactive lanes pass active=false and zero data) because of the cross-lane reductions.
// Writes the outlier values and the group scales; returns the packed word in lo/hi.
template <int BITS>
__device__ __forceinline__ void encode_chan(const uint4* raw, bool active, int c, int CPS, int lpg, const ChanArgs& a,
                                            uint16_t* vals_row, uint16_t* scales_row, uint32_t& lo, uint32_t& hi) {
  constexpr int NSEG = Q<BITS>::NSEG;
  lo = 0; hi = 0;
#pragma unroll
  for (int i = 0; i < NSEG; ++i) {
    float v[8];
    unpack8(raw[i], v);
    const int cg = i * CPS + c;                        // chunk index within the full row
    const uint32_t p = active ? a.plan[cg] : 0u;
    const uint32_t m8 = p & 0xFFu;
    if (m8) {                                          // rare: ~k/(H/8) of the chunks
      const int first = (int)(p >> 16);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if ((m8 >> j) & 1u) {
          vals_row[first + __popc(m8 & ((1u << j) - 1u))] = raw16(raw[i], j);
          v[j] = 0.f;                                  // x - x*mask is an exact zero
        }
      }
    }
    float mx = v[0], mn = v[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) { mx = v[j] > mx ? v[j] : mx; mn = v[j] < mn ? v[j] : mn; }
    mx = group_reduce_rt(mx, lpg, OpMax());
    mn = group_reduce_rt(mn, lpg, OpMin());
    const float s = bfr(bfr(mx - mn) * Q<BITS>::INV_LEVELS);   // == bf16(bf16(max-min)/levels), see make_recip
    if (active && (c & (lpg - 1)) == 0) scales_row[cg >> a.chunk_to_group_shift] = f_to_bf(s);
    const Recip k = make_recip(s);
    float q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = quant1<BITS>(v[j], k);
    put_codes<BITS>(q, i, lo, hi);
  }
}

// Decode chunk c of segment i of one row to 8 floats holding bf16 values.
template <int BITS>
__device__ __forceinline__ void decode_chan(uint32_t lo, uint32_t hi, int i, int c, int CPS, const ChanArgs& a,
                                            const uint16_t* vals_row, const uint16_t* scales_row, float (&v)[8]) {
  const int cg = i * CPS + c;
  const float s = bf_to_f(scales_row[cg >> a.chunk_to_group_shift]);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = bfr(get_code<BITS>(lo, hi, i, j) * s) + 0.f;   // 0 + d: a -0 becomes +0
  const uint32_t p = a.plan[cg];
  const uint32_t m8 = p & 0xFFu;
  if (m8) {
    const int first = (int)(p >> 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((m8 >> j) & 1u) {
        const float o = bf_to_f(vals_row[first + __popc(m8 & ((1u << j) - 1u))]) + 0.f;
        v[j] = bfr(o + v[j]);                          // (0 + outlier) + dequant; dequant is 0 here
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// threshold mode
// ------------------------------------------------------------------------------------------------
// Encode; returns the number of outliers among the thread's elements.  No cross-lane work.
template <int BITS, bool PERCHAN>
__device__ __forceinline__ int encode_thr(const uint4* raw, int c, int CPS, int64_t H, int64_t s_pos,
                                          const ThrArgs& a, uint32_t& lo, uint32_t& hi) {
  constexpr int NSEG = Q<BITS>::NSEG;
  lo = 0; hi = 0;
  int hot = 0;
#pragma unroll
  for (int i = 0; i < NSEG; ++i) {
    float v[8];
    unpack8(raw[i], v);
    const int64_t col = ((int64_t)i * CPS + c) * 8;
    if (a.rank > 0) {
      float b[8];
      base8(a, s_pos, col, H, b);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = bfr(v[j] - b[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool h = __builtin_fabsf(v[j]) > a.thr;
      hot += h ? 1 : 0;
      v[j] = h ? 0.f : v[j];
    }
    float q[8];
    if (PERCHAN) {
      const uint4 sr = *reinterpret_cast<const uint4*>(a.scale + s_pos * a.sst + col);   // ssc == 1
      float sv[8];
      unpack8(sr, sv);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        Recip k; k.s = sv[j]; k.r = 0.f; k.exact = true;
        q[j] = quant1<BITS>(v[j], k);
      }
    } else {
      const Recip k = make_recip(bf_to_f(a.scale[s_pos * a.sst]));
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = quant1<BITS>(v[j], k);
    }
    put_codes<BITS>(q, i, lo, hi);
  }
  return hot;
}

// Decode chunk c of segment i WITHOUT the outliers: v = bf16(bf16(base + 0) + dequant).  The callers add the
// row's CSR outliers afterwards (at those positions dequant is 0, so x_hat = bf16(base + outlier)).
template <int BITS, bool PERCHAN>
__device__ __forceinline__ void decode_thr(uint32_t lo, uint32_t hi, int i, int c, int CPS, int64_t H, int64_t s_pos,
                                           const ThrArgs& a, float (&v)[8], float (&base)[8]) {
  const int64_t col = ((int64_t)i * CPS + c) * 8;
  if (a.rank > 0) {
    base8(a, s_pos, col, H, base);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) base[j] = 0.f;
  }
  if (PERCHAN) {
    const uint4 sr = *reinterpret_cast<const uint4*>(a.scale + s_pos * a.sst + col);
    float sv[8];
    unpack8(sr, sv);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = bfr((base[j] + 0.f) + bfr(get_code<BITS>(lo, hi, i, j) * sv[j]));
  } else {
    const float s = bf_to_f(a.scale[s_pos * a.sst]);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = bfr((base[j] + 0.f) + bfr(get_code<BITS>(lo, hi, i, j) * s));
  }
}

}  // namespace hyc
