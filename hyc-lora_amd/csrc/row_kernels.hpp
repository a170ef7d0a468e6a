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
// One segment-chunk of the encoder: 8 activations (already as floats, `rawseg` = their bf16 bits) -> 8 code bytes.
// plan word `p` (see hyc_desc.chan_plan) marks the outlier channels of the chunk; their values go to vals_row and
// they are quantised as exact zeros.  Cross-lane: every lane of the wave must take part.
// Returns the group scale; the caller stores it from the first lane of each group.
// RULE: the group scale rule, SCALE_RANGE / SCALE_ABSMAX, or SCALE_RUNTIME = decided by the flag `absmax` (uniform).
constexpr int SCALE_RANGE = 0, SCALE_ABSMAX = 1, SCALE_RUNTIME = -1;
template <int BITS, int LPGT, int RULE = SCALE_RUNTIME>
__device__ __forceinline__ float quant_seg(float (&v)[8], int lpg, uint32_t& cl, uint32_t& ch, bool absmax);

// LPGT: lanes per scale group when known at compile time, 0 = use the runtime value `lpg`.
template <int BITS, int LPGT = 0>
__device__ __forceinline__ float encode_seg(const uint4& rawseg, float (&v)[8], uint32_t p, int lpg, uint16_t* vals_row,
                                            uint32_t& cl, uint32_t& ch, bool absmax) {
  if (__builtin_expect((p & 0xFFu) != 0, 0)) {         // rare: ~k/(H/8) of the chunks
    const uint32_t m8 = p & 0xFFu;
    const int first = (int)(p >> 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((m8 >> j) & 1u) {
        vals_row[first + __popc(m8 & ((1u << j) - 1u))] = raw16(rawseg, j);
        v[j] = 0.f;                                    // x - x*mask is an exact zero
      }
    }
  }
  return quant_seg<BITS, LPGT>(v, lpg, cl, ch, absmax);
}

// group statistics -> scale -> 8 code bytes, no outlier handling (the caller has zeroed the outlier channels).
//   range rule    s = bf16(bf16(max - min) / (2^b - 1))      the reference's formula, compress_function.py:328-334
//   abs-max rule  s = bf16(bf16(2 max|x|) / (2^b - 1))       the same formula over the interval made symmetric about 0,
//                 [-max|x|, max|x|]: no element is off by more than half a step, one butterfly instead of two
//                 (1-bit codes, {-1, 0}: s = max|x|)
// Both quotients are formed as a product with the rounded reciprocal: the dividend is a bf16 value (an integer below
// 256 times a power of two) and the divisor an integer below 256, so the exact quotient never lies within 2^-17
// (relative) of a bf16 rounding boundary, far more than the 2^-23 the product can be off by.
template <int BITS, int LPGT, int RULE>
__device__ __forceinline__ float quant_seg(float (&v)[8], int lpg, uint32_t& cl, uint32_t& ch, bool absmax) {
  float s;
  if (RULE == SCALE_ABSMAX || (RULE == SCALE_RUNTIME && absmax)) {
    float am = __builtin_elementwise_maximum(__builtin_elementwise_maximum(__builtin_fabsf(v[0]), __builtin_fabsf(v[1])), __builtin_fabsf(v[2]));
    am = __builtin_elementwise_maximum(__builtin_elementwise_maximum(am, __builtin_fabsf(v[3])), __builtin_fabsf(v[4]));
    am = __builtin_elementwise_maximum(__builtin_elementwise_maximum(am, __builtin_fabsf(v[5])), __builtin_fabsf(v[6]));
    am = __builtin_elementwise_maximum(am, __builtin_fabsf(v[7]));
    if (LPGT > 0) am = group_max_nonneg<LPGT>(am);
    else am = group_max_nonneg_rt(am, lpg);
    s = BITS == 1 ? am : bfr((am + am) * Q<BITS>::INV_LEVELS);
  } else {
    float mx = __builtin_elementwise_maximum(__builtin_elementwise_maximum(v[0], v[1]), v[2]);
    float mn = __builtin_elementwise_minimum(__builtin_elementwise_minimum(v[0], v[1]), v[2]);
    mx = __builtin_elementwise_maximum(__builtin_elementwise_maximum(mx, v[3]), v[4]);
    mn = __builtin_elementwise_minimum(__builtin_elementwise_minimum(mn, v[3]), v[4]);
    mx = __builtin_elementwise_maximum(__builtin_elementwise_maximum(mx, v[5]), v[6]);
    mn = __builtin_elementwise_minimum(__builtin_elementwise_minimum(mn, v[5]), v[6]);
    mx = __builtin_elementwise_maximum(mx, v[7]);
    mn = __builtin_elementwise_minimum(mn, v[7]);
    if (LPGT > 0) {
      group_maxmin<LPGT>(mx, mn);
    } else {
      mx = group_reduce_rt(mx, lpg, OpMax());
      mn = group_reduce_rt(mn, lpg, OpMin());
    }
    s = bfr(bfr(mx - mn) * Q<BITS>::INV_LEVELS);
  }
  codes8<BITS>(v, s, cl, ch);
  return s;
}

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
    uint32_t cl, ch;
    const float s = encode_seg<BITS>(raw[i], v, p, lpg, vals_row, cl, ch, a.absmax != 0);
    if (active && (c & (lpg - 1)) == 0) scales_row[cg >> a.chunk_to_group_shift] = f_to_bf(s);
    if (BITS == 8) { lo = cl; hi = ch; }
    else { lo |= cl << (i * BITS); hi |= ch << (i * BITS); }
  }
}

// Decode segment i of a packed word to 8 bf16 values (four packed pairs), given the group scale and the chunk's
// plan word.
template <int BITS>
__device__ __forceinline__ uint4 decode_seg(uint32_t lo, uint32_t hi, int i, float s, uint32_t p, const uint16_t* vals_row) {
  uint4 r = dequant8<BITS>(lo, hi, i, s);
  if (__builtin_expect((p & 0xFFu) != 0, 0)) {
    const uint32_t m8 = p & 0xFFu;
    const int first = (int)(p >> 16);
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((m8 >> j) & 1u) {
        // (0 + outlier) + dequant, where dequant is the zero the outlier position was quantised to
        const float o = bf_to_f(vals_row[first + __popc(m8 & ((1u << j) - 1u))]) + 0.f;
        const float d = (j & 1) ? bf_hi(w[j >> 1]) : bf_lo(w[j >> 1]);
        const uint32_t nb = f_to_bf(o + d);
        w[j >> 1] = (j & 1) ? ((w[j >> 1] & 0x0000FFFFu) | (nb << 16)) : ((w[j >> 1] & 0xFFFF0000u) | nb);
      }
    }
    r = make_uint4(w[0], w[1], w[2], w[3]);
  }
  return r;
}

// ---- outliers without per-element branches (fast kernels) -----------------------------------------------------
// The outlier channel set is static, so what a thread has to do about outliers is the same for every row and is
// worked out once from the plan words.
//   decode side: the packed codes of outlier channels decode to 0 (they were quantised as zeros).  The thread
//     requests the first two outlier values of each of its chunks together with the row's other loads and splices
//     them into the decoded chunk with four byte-permutes whose selectors are per-lane constants.  Chunks with
//     more than two outlier channels are finished by splice_more(): a loop whose trip count is the same for the
//     whole wave and zero unless one of its lanes owns such a chunk.
//   encode side: the outlier channels are zeroed with precomputed AND masks, and the side tensor vals[m, :] is
//     filled by the first k threads of the workgroup straight from x (gather through L1/L2, coalesced store).

// v_perm selectors that put outlier j0 (bytes 4-5 of the outlier pair word) and, if has1, j1 (bytes 6-7) into the
// four bf16-pair words of a decoded chunk; bytes 0-3 keep the decoded word
__device__ __forceinline__ void splice_selectors(bool has0, int j0, bool has1, int j1, uint32_t (&sel)[4]) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint32_t q = 0x03020100u;
    if (has0 && (j0 >> 1) == w) q = (j0 & 1) ? ((q & 0x0000FFFFu) | 0x05040000u) : ((q & 0xFFFF0000u) | 0x00000504u);
    if (has1 && (j1 >> 1) == w) q = (j1 & 1) ? ((q & 0x0000FFFFu) | 0x07060000u) : ((q & 0xFFFF0000u) | 0x00000706u);
    sel[w] = q;
  }
}
// The reconstruction is (0 + outlier) + dequant(zero code): a -0 outlier comes out as +0, and a group whose scale
// is inf/NaN is NaN at the outlier channels too.
// SIGNED_ZERO = false leaves a -0 outlier as it is: for consumers that only multiply and add the restored value
// (the weight gradient) the sign of a zero cannot reach the result.
template <bool SIGNED_ZERO = true>
__device__ __forceinline__ uint4 splice_pair(const uint4& r, const uint32_t (&sel)[4], uint32_t o0, uint32_t o1, float s) {
  if (SIGNED_ZERO) {
    o0 = o0 == 0x8000u ? 0u : o0;
    o1 = o1 == 0x8000u ? 0u : o1;
  }
  uint32_t oo = o0 | (o1 << 16);
  oo = (0.f * s == 0.f) ? oo : 0x7FC07FC0u;
  return make_uint4(__builtin_amdgcn_perm(oo, r.x, sel[0]), __builtin_amdgcn_perm(oo, r.y, sel[1]),
                    __builtin_amdgcn_perm(oo, r.z, sel[2]), __builtin_amdgcn_perm(oo, r.w, sel[3]));
}

template <int NSEG>
struct ChunkOutliers {
  uint32_t sel[NSEG][4];   // selectors of the first outlier pair
  uint32_t m8[NSEG];       // outlier bit mask of the chunk
  uint32_t vb[NSEG];       // byte offset of the chunk's first outlier in vals[m, :]
  bool has0[NSEG], has1[NSEG];
  int more_pairs;          // wave-uniform: outlier pairs beyond the first in the fullest chunk of the wave (0..3)

  __device__ __forceinline__ void init(const uint32_t (&plan)[NSEG]) {
    int most = 0;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      m8[i] = plan[i] & 0xFFu;
      vb[i] = (plan[i] >> 16) * 2u;
      const int n = __popc(m8[i]);
      has0[i] = n > 0; has1[i] = n > 1;
      const int j0 = m8[i] ? __ffs(m8[i]) - 1 : 0;
      const uint32_t rest = m8[i] & (m8[i] - 1);
      const int j1 = rest ? __ffs(rest) - 1 : 0;
      splice_selectors(has0[i], j0, has1[i], j1, sel[i]);
      most = n > most ? n : most;
    }
    more_pairs = (__ballot(most > 2) != 0) + (__ballot(most > 4) != 0) + (__ballot(most > 6) != 0);
  }
  // AND masks that zero the outlier channels in the four bf16-pair words of chunk i
  __device__ __forceinline__ void keep_masks(int i, uint32_t (&km)[4]) const {
#pragma unroll
    for (int w = 0; w < 4; ++w)
      km[w] = (((m8[i] >> (2 * w)) & 1u) ? 0u : 0x0000FFFFu) | (((m8[i] >> (2 * w + 1)) & 1u) ? 0u : 0xFFFF0000u);
  }
  // request the first two outlier values of every chunk from vals[m, :] (no wait here)
  __device__ __forceinline__ void request(const uint16_t* vals_row, uint32_t (&o0)[NSEG], uint32_t (&o1)[NSEG]) const {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      o0[i] = 0; o1[i] = 0;
      const char* b = reinterpret_cast<const char*>(vals_row);        // uniform base + 32-bit lane offset
      if (has0[i]) o0[i] = *reinterpret_cast<const uint16_t*>(b + vb[i]);
      if (has1[i]) o1[i] = *reinterpret_cast<const uint16_t*>((b + 2) + vb[i]);
    }
  }
  __device__ __forceinline__ uint4 splice(int i, const uint4& r, uint32_t o0, uint32_t o1, float s) const {
    return splice_pair(r, sel[i], o0, o1, s);
  }
  // the same for consumers that are indifferent to the sign of a zero
  __device__ __forceinline__ uint4 splice_value(int i, const uint4& r, uint32_t o0, uint32_t o1) const {
    return splice_pair<false>(r, sel[i], o0, o1, 1.f);
  }
};

// Outlier pairs 1..more_pairs of a chunk (plan word p); `ok` = the row exists.  Loads and waits in place: only
// waves that own a chunk with more than two outlier channels come here.
__device__ __forceinline__ uint4 splice_more(uint4 r, int more_pairs, uint32_t p, const uint16_t* vals_row, bool ok, float s) {
  uint32_t m = p & 0xFFu;
  int at = (int)(p >> 16);
  for (int q = 1; q <= more_pairs; ++q) {
    m &= m - 1; m &= m - 1;                              // drop the pair already spliced
    at += 2;
    if (m != 0 && ok) {
      const uint32_t rest = m & (m - 1);
      uint32_t sel[4];
      splice_selectors(true, __ffs(m) - 1, rest != 0, rest ? __ffs(rest) - 1 : 0, sel);
      const uint32_t o0 = vals_row[at], o1 = rest ? vals_row[at + 1] : 0u;
      r = splice_pair(r, sel, o0, o1, s);
    }
  }
  return r;
}

// Decode chunk c of segment i of one row (loads the scale and the plan word itself).
template <int BITS>
__device__ __forceinline__ uint4 decode_chan_pk(uint32_t lo, uint32_t hi, int i, int c, int CPS, const ChanArgs& a,
                                                const uint16_t* vals_row, const uint16_t* scales_row) {
  const int cg = i * CPS + c;
  return decode_seg<BITS>(lo, hi, i, bf_to_f(scales_row[cg >> a.chunk_to_group_shift]), a.plan[cg], vals_row);
}

template <int BITS>
__device__ __forceinline__ void decode_chan(uint32_t lo, uint32_t hi, int i, int c, int CPS, const ChanArgs& a,
                                            const uint16_t* vals_row, const uint16_t* scales_row, float (&v)[8]) {
  unpack8(decode_chan_pk<BITS>(lo, hi, i, c, CPS, a, vals_row, scales_row), v);
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
    if (PERCHAN) {
      float q[8];
      const uint4 sr = *reinterpret_cast<const uint4*>(a.scale + s_pos * a.sst + col);   // ssc == 1
      float sv[8];
      unpack8(sr, sv);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        Recip k; k.s = sv[j]; k.r = 0.f; k.exact = true;
        q[j] = quant1<BITS>(v[j], k);
      }
      put_codes<BITS>(q, i, lo, hi);
    } else {
      uint32_t cl, ch;
      codes8<BITS>(v, bf_to_f(a.scale[s_pos * a.sst]), cl, ch);
      if (BITS == 8) { lo = cl; hi = ch; }
      else { lo |= cl << (i * BITS); hi |= ch << (i * BITS); }
    }
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
