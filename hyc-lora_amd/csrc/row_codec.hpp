// Device-side building blocks shared by every kernel of the library (gfx950, wave64).
//
// Thread <-> data mapping of one row of H channels at `BITS` bits per code:
//   the row is cut into NSEG = 8/BITS segments of SEG = H/NSEG channels (the reference's packing,
//   operators/compress_function.py:175-197).  A segment is CPS = SEG/8 chunks of 8 channels.  In
//   iteration `it` thread t owns chunk c = it*blockDim.x + t of EVERY segment: NSEG 16-byte loads of
//   bf16 activations give exactly the 8 packed bytes [8c, 8c+8) of the stored row - one 8-byte store.
//   A scale group of G channels is G/8 consecutive chunks = G/8 consecutive lanes (LPG), so group
//   min/max are DPP butterflies inside a 16-lane row and never touch LDS.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hyc {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ __forceinline__ float bf_to_f(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// two floats -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  floatx2_t v = {lo, hi};
  bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint16_t f_to_bf(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}
// round an fp32 value to the nearest bf16 and return it as fp32
__device__ __forceinline__ float bfr(float f) { return (float)((__bf16)f); }

// 8 consecutive bf16 <-> 8 floats
__device__ __forceinline__ void unpack8(const uint4& r, float (&v)[8]) {
  v[0] = bf_lo(r.x); v[1] = bf_hi(r.x); v[2] = bf_lo(r.y); v[3] = bf_hi(r.y);
  v[4] = bf_lo(r.z); v[5] = bf_hi(r.z); v[6] = bf_lo(r.w); v[7] = bf_hi(r.w);
}
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  uint4 r;
  r.x = pack_bf16(v[0], v[1]); r.y = pack_bf16(v[2], v[3]);
  r.z = pack_bf16(v[4], v[5]); r.w = pack_bf16(v[6], v[7]);
  return r;
}

// 16-byte store of a streaming output (written once, not read again by this kernel): bypasses cache allocation.
// Measured on MI355X: with loads in flight, plain 16-byte stores reach ~4.1 TB/s, these ~5.4 TB/s.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_stream(uint16_t* p, const uint4& v) {
  const u32x4_t t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(p));
}

// ---- buffer addressing ----------------------------------------------------------------------------
// A resource is (base, bytes); a lane whose offset is at or beyond `bytes` reads zeros / has its store dropped
// instead of faulting.  Kernels use that to keep their memory instructions unconditional: rows past the end get a
// resource of zero bytes, lanes without data the offset NOWHERE.  (Straight-line code lets the compiler count the
// operations in flight exactly, so it waits for the one it needs and no more.)
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
constexpr uint32_t NOWHERE = 0x80000000u;                // beyond any resource (sizes stay below 2 GiB)
__device__ __forceinline__ BufferRsrc make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 load_b128(BufferRsrc r, uint32_t off) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_b64(BufferRsrc r, uint32_t off) {
  const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
  return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t load_b32(BufferRsrc r, uint32_t off) {
  return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0);
}
__device__ __forceinline__ uint32_t load_b16(BufferRsrc r, uint32_t off) {
  return (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0);
}
// streaming 16-byte store (written once, not read again by this kernel)
__device__ __forceinline__ void store_b128_stream(BufferRsrc r, uint32_t off, const uint4& v) {
  const u32x4_t t = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(t, r, (int)off, 0, 2);
}
__device__ __forceinline__ void store_b64(BufferRsrc r, uint32_t off, uint32_t lo, uint32_t hi) {
  const u32x2_t t = {lo, hi};
  __builtin_amdgcn_raw_buffer_store_b64(t, r, (int)off, 0, 0);
}
__device__ __forceinline__ void store_b32(BufferRsrc r, uint32_t off, uint32_t v) {
  __builtin_amdgcn_raw_buffer_store_b32(v, r, (int)off, 0, 0);
}
__device__ __forceinline__ void store_b16(BufferRsrc r, uint32_t off, uint16_t v) {
  __builtin_amdgcn_raw_buffer_store_b16((short)v, r, (int)off, 0, 0);
}
// 16 bytes per lane from memory straight into LDS: lane i of the wave lands at `lds_wave_base` + 16 i
__device__ __forceinline__ void load_b128_to_lds(BufferRsrc r, uint32_t off, void* lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)lds_wave_base, 16, (int)off, 0, 0, 0);
}

// ---- cross-lane -------------------------------------------------------------------------------
// value of another lane of the same 16-lane row.  OLD_ZERO: lanes without a source read 0 (lets the compiler fold
// the move into v_add_f32_dpp).
template <int CTRL, bool OLD_ZERO>
__device__ __forceinline__ float dpp_f(float v) {
  const int self = __builtin_bit_cast(int, v);
  if (OLD_ZERO) return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, self, CTRL, 0xF, 0xF, false));
  // every pattern used here (quad_perm, row_half_mirror, row_mirror) has a valid source lane for every lane, so the
  // previous content of the destination is never read: leave it undefined (a single v_mov_b32_dpp)
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(self, CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float xor_lane(float v, int m) { return __shfl_xor(v, m, 64); }

struct OpMax {
  static constexpr bool ZERO = false;
  __device__ __forceinline__ float operator()(float a, float b) const { return __builtin_elementwise_maximum(a, b); }
};
struct OpMin {
  static constexpr bool ZERO = false;
  __device__ __forceinline__ float operator()(float a, float b) const { return __builtin_elementwise_minimum(a, b); }
};
struct OpAdd {
  static constexpr bool ZERO = true;
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

// butterfly over LPG consecutive lanes (LPG a power of two <= 64); every lane of the group gets the result.
// Must be executed by all lanes of the wave (callers feed neutral values from lanes without data).
template <int LPG, typename Op>
__device__ __forceinline__ float group_reduce(float v, Op op) {
  if (LPG >= 2) v = op(v, dpp_f<0xB1, Op::ZERO>(v));   // quad_perm [1,0,3,2]
  if (LPG >= 4) v = op(v, dpp_f<0x4E, Op::ZERO>(v));   // quad_perm [2,3,0,1]
  if (LPG >= 8) v = op(v, dpp_f<0x141, Op::ZERO>(v));  // row_half_mirror
  if (LPG >= 16) v = op(v, dpp_f<0x140, Op::ZERO>(v)); // row_mirror
  if (LPG >= 32) v = op(v, xor_lane(v, 16));
  if (LPG >= 64) v = op(v, xor_lane(v, 32));
  return v;
}
// max of `mx` and min of `mn` over LPG lanes, the two butterflies interleaved so that neither waits on the
// read-after-write distance a DPP source needs
template <int LPG>
__device__ __forceinline__ void group_maxmin(float& mx, float& mn) {
#define HYC_STEP(CTRL)                                                     \
  {                                                                        \
    const float a_ = dpp_f<CTRL, false>(mx), b_ = dpp_f<CTRL, false>(mn);  \
    mx = __builtin_elementwise_maximum(mx, a_);                            \
    mn = __builtin_elementwise_minimum(mn, b_);                            \
  }
  if (LPG >= 2) HYC_STEP(0xB1)
  if (LPG >= 4) HYC_STEP(0x4E)
  if (LPG >= 8) HYC_STEP(0x141)
  if (LPG >= 16) HYC_STEP(0x140)
#undef HYC_STEP
  if (LPG >= 32) { mx = __builtin_elementwise_maximum(mx, xor_lane(mx, 16)); mn = __builtin_elementwise_minimum(mn, xor_lane(mn, 16)); }
  if (LPG >= 64) { mx = __builtin_elementwise_maximum(mx, xor_lane(mx, 32)); mn = __builtin_elementwise_minimum(mn, xor_lane(mn, 32)); }
}
// Maximum of a NON-NEGATIVE value over LPG consecutive lanes.  Non-negative floats order like their bit patterns, and
// an integer maximum takes the other lane's value as a DPP operand (one v_max_u32_dpp per step); the float maximum
// needs a v_mov_b32_dpp in front of every v_max_f32, because its operands have to be canonicalised first.
template <int CTRL>
__device__ __forceinline__ uint32_t umax_dpp(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);   // (every lane has a source; 0 is max's identity)
  return v > o ? v : o;
}
template <int LPG>
__device__ __forceinline__ float group_max_nonneg(float v) {
  uint32_t b = __float_as_uint(v);
  if (LPG >= 2) b = umax_dpp<0xB1>(b);     // quad_perm [1,0,3,2]
  if (LPG >= 4) b = umax_dpp<0x4E>(b);     // quad_perm [2,3,0,1]
  if (LPG >= 8) b = umax_dpp<0x141>(b);    // row_half_mirror
  if (LPG >= 16) b = umax_dpp<0x140>(b);   // row_mirror
  if (LPG >= 32) { const uint32_t o = (uint32_t)__shfl_xor((int)b, 16, 64); b = b > o ? b : o; }
  if (LPG >= 64) { const uint32_t o = (uint32_t)__shfl_xor((int)b, 32, 64); b = b > o ? b : o; }
  return __uint_as_float(b);
}
__device__ __forceinline__ float group_max_nonneg_rt(float v, int lpg) {
  uint32_t b = __float_as_uint(v);
  b = umax_dpp<0xB1>(b);
  b = umax_dpp<0x4E>(b);
  if (lpg >= 8) b = umax_dpp<0x141>(b);
  if (lpg >= 16) b = umax_dpp<0x140>(b);
  if (lpg >= 32) { const uint32_t o = (uint32_t)__shfl_xor((int)b, 16, 64); b = b > o ? b : o; }
  if (lpg >= 64) { const uint32_t o = (uint32_t)__shfl_xor((int)b, 32, 64); b = b > o ? b : o; }
  return __uint_as_float(b);
}
// runtime-width variant (lpg in {4, 8, 16, 32, 64}; the branches are uniform)
template <typename Op>
__device__ __forceinline__ float group_reduce_rt(float v, int lpg, Op op) {
  v = op(v, dpp_f<0xB1, Op::ZERO>(v));
  v = op(v, dpp_f<0x4E, Op::ZERO>(v));
  if (lpg >= 8) v = op(v, dpp_f<0x141, Op::ZERO>(v));
  if (lpg >= 16) v = op(v, dpp_f<0x140, Op::ZERO>(v));
  if (lpg >= 32) v = op(v, xor_lane(v, 16));
  if (lpg >= 64) v = op(v, xor_lane(v, 32));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) { return group_reduce<64>(v, OpAdd()); }

// sum over the whole workgroup; `red` is LDS scratch of >= 16 floats per reduction slot.
// All threads return the total.  Contains two barriers.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  __syncthreads();
  return t;
}

// ---- quantise one chunk -------------------------------------------------------------------------
template <int BITS>
struct Q {
  static constexpr int NSEG = 8 / BITS;
  static constexpr int OFF = 1 << (BITS - 1);
  static constexpr float LO = -(float)OFF;
  static constexpr float HI = (float)(OFF - 1);
  static constexpr float INV_LEVELS = 1.0f / (float)((1 << BITS) - 1);
  static constexpr uint32_t CODE_MASK = (1u << BITS) - 1;
};

// reciprocal used for q = bf16(x / s).  For bf16 x and s in the normal range the exact quotient is a
// ratio of two integers below 256, which can never sit closer than 2^-17 (relative) to a bf16
// rounding boundary, so bf16(x * fl(1/s)) equals bf16(fl(x / s)); outside that range fall back to the
// IEEE division (`exact` = true).
struct Recip {
  float r;
  float s;
  bool exact;
};
__device__ __forceinline__ Recip make_recip(float s) {
  Recip k;
  k.s = s;
  k.exact = !(s > 1e-30f && s < 1e30f);   // also true for negative, zero, NaN scales
  k.r = 1.0f / s;
  return k;
}
// signed code q (as float, already clamped) of one element.  x / 0 = +-inf clamps like any large quotient;
// 0 / 0 = NaN, whose integer cast the reference leaves undefined, is given q = 0 (code = offset).
template <int BITS>
__device__ __forceinline__ float quant1(float x, const Recip& k) {
  float t = k.exact ? (x / k.s) : (x * k.r);
  t = __builtin_rintf(bfr(t));
  t = (t != t) ? 0.f : t;
  return __builtin_fminf(__builtin_fmaxf(t, Q<BITS>::LO), Q<BITS>::HI);
}

// 8 signed codes -> OR into the packed 8-byte word at bit field `seg`
template <int BITS>
__device__ __forceinline__ void put_codes(const float (&q)[8], int seg, uint32_t& lo, uint32_t& hi) {
  if (BITS == 8) {
    lo = ((uint32_t)(int)q[0] & 0xFF) | (((uint32_t)(int)q[1] & 0xFF) << 8) | (((uint32_t)(int)q[2] & 0xFF) << 16) |
         (((uint32_t)(int)q[3] & 0xFF) << 24);
    hi = ((uint32_t)(int)q[4] & 0xFF) | (((uint32_t)(int)q[5] & 0xFF) << 8) | (((uint32_t)(int)q[6] & 0xFF) << 16) |
         (((uint32_t)(int)q[7] & 0xFF) << 24);
  } else {
    const int sh = seg * BITS;
    uint32_t a = (uint32_t)((int)q[0] + Q<BITS>::OFF) | ((uint32_t)((int)q[1] + Q<BITS>::OFF) << 8) |
                 ((uint32_t)((int)q[2] + Q<BITS>::OFF) << 16) | ((uint32_t)((int)q[3] + Q<BITS>::OFF) << 24);
    uint32_t b = (uint32_t)((int)q[4] + Q<BITS>::OFF) | ((uint32_t)((int)q[5] + Q<BITS>::OFF) << 8) |
                 ((uint32_t)((int)q[6] + Q<BITS>::OFF) << 16) | ((uint32_t)((int)q[7] + Q<BITS>::OFF) << 24);
    lo |= a << sh;
    hi |= b << sh;
  }
}

// signed value (code - offset, or the int8 itself) of element j of segment `seg` in a packed word
template <int BITS>
__device__ __forceinline__ float get_code(uint32_t lo, uint32_t hi, int seg, int j) {
  const uint32_t w = (j < 4) ? lo : hi;
  const int byte = (int)((w >> ((j & 3) * 8)) & 0xFF);
  if (BITS == 8) return (float)(int)(int8_t)byte;
  return (float)((int)((byte >> (seg * BITS)) & Q<BITS>::CODE_MASK) - Q<BITS>::OFF);
}

// ---- lean forms used by the channel-mode kernels ------------------------------------------------
// Same arithmetic as quant1 / put_codes / get_code above, arranged for few VALU operations per element.

// Code bytes of 8 elements: byte j of {lo, hi} = q_j + OFF (BITS < 8) or the int8 q_j (BITS == 8).
//   fast path  t = bf16(x * r), r = 1/s refined to full fp32 precision (see Recip); the clamp uses v_med3 and
//              the round-half-even + offset + float->int conversion are one add of 1.5*2^23 + OFF, which leaves
//              q + OFF in the low mantissa byte.  clamp(rint(t)) == rint(clamp(t)) because the bounds are integers.
//   slow path  scales outside (1e-30, 1e30), zero included: IEEE division, NaN (0/0) -> q = 0.
template <int BITS>
__device__ __forceinline__ void codes8(const float (&v)[8], float s, uint32_t& lo, uint32_t& hi) {
  // the added constant must stay even, or the tie-breaking of the half-even rounding flips: 1-bit codes
  // (OFF = 1) are formed with an offset of 2 and corrected after the gather
  constexpr int OFF_EVEN = (BITS == 8) ? 0 : ((Q<BITS>::OFF + 1) & ~1);
  constexpr float MAGIC = 12582912.0f + (float)OFF_EVEN;
  uint32_t u[8];
  if (__builtin_expect(s > 1e-30f && s < 1e30f, 1)) {
    float r = __builtin_amdgcn_rcpf(s);
    r = __builtin_fmaf(__builtin_fmaf(-s, r, 1.0f), r, r);
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      const uint32_t pk = pack_bf16(v[j] * r, v[j + 1] * r);
      const float c0 = __builtin_amdgcn_fmed3f(bf_lo(pk), Q<BITS>::LO, Q<BITS>::HI);
      const float c1 = __builtin_amdgcn_fmed3f(bf_hi(pk), Q<BITS>::LO, Q<BITS>::HI);
      u[j] = __float_as_uint(c0 + MAGIC);
      u[j + 1] = __float_as_uint(c1 + MAGIC);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float t = __builtin_rintf(bfr(v[j] / s));
      t = (t != t) ? 0.f : t;
      t = __builtin_fminf(__builtin_fmaxf(t, Q<BITS>::LO), Q<BITS>::HI);
      u[j] = __float_as_uint(t + MAGIC);
    }
  }
  // gather byte 0 of four words into one
  const uint32_t p01 = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u);
  const uint32_t p23 = __builtin_amdgcn_perm(u[3], u[2], 0x0c0c0400u);
  const uint32_t p45 = __builtin_amdgcn_perm(u[5], u[4], 0x0c0c0400u);
  const uint32_t p67 = __builtin_amdgcn_perm(u[7], u[6], 0x0c0c0400u);
  lo = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
  hi = __builtin_amdgcn_perm(p67, p45, 0x05040100u);
  if (BITS != 8 && OFF_EVEN != Q<BITS>::OFF) {
    lo -= (uint32_t)(OFF_EVEN - Q<BITS>::OFF) * 0x01010101u;
    hi -= (uint32_t)(OFF_EVEN - Q<BITS>::OFF) * 0x01010101u;
  }
}

// The eight byte values of two words as floats.  Codes below 16 (1-, 2- and 4-bit) go two per instruction: a byte
// below 17 read as an FP8 number (E4M3, bias 7) is that integer times 2^-9 (the exponent fields 0 and 1 share one
// step), and the scaled packed conversion multiplies by a power of two on its way (it takes the exponent of its scale
// operand), so with 2^9 the two bytes of a half-word come out as the floats of their integer values, exactly.
template <int BITS>
__device__ __forceinline__ void codes8_to_float(uint32_t a, uint32_t b, float (&c)[8]) {
  if (BITS <= 4) {
    const floatx2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(a, 512.f, false);
    const floatx2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(a, 512.f, true);
    const floatx2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(b, 512.f, false);
    const floatx2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(b, 512.f, true);
    c[0] = p0.x; c[1] = p0.y; c[2] = p1.x; c[3] = p1.y; c[4] = p2.x; c[5] = p2.y; c[6] = p3.x; c[7] = p3.y;
  } else {
    c[0] = (float)(a & 0xFFu); c[1] = (float)((a >> 8) & 0xFFu); c[2] = (float)((a >> 16) & 0xFFu); c[3] = (float)(a >> 24);
    c[4] = (float)(b & 0xFFu); c[5] = (float)((b >> 8) & 0xFFu); c[6] = (float)((b >> 16) & 0xFFu); c[7] = (float)(b >> 24);
  }
}

// Dequantised values of segment `seg` of a packed word, as four packed bf16 pairs:
// x_hat = bf16((code - OFF) * s); (code - OFF) * s is exact in fp32, so one fma and one rounding.
template <int BITS>
__device__ __forceinline__ uint4 dequant8(uint32_t lo, uint32_t hi, int seg, float s) {
  constexpr uint32_t REP = (BITS == 8) ? 0x80808080u : Q<BITS>::CODE_MASK * 0x01010101u;
  uint32_t a, b;
  if (BITS == 8) { a = lo ^ REP; b = hi ^ REP; }             // int8 -> biased unsigned (q + 128)
  else { a = (lo >> (seg * BITS)) & REP; b = (hi >> (seg * BITS)) & REP; }
  // opaque from here on: the codes of a word are then converted straight from its bytes (left to itself the
  // compiler extracts every field from the packed word first: two instructions per code)
  asm volatile("" : "+v"(a), "+v"(b));
  float c[8];
  codes8_to_float<BITS>(a, b, c);
  constexpr float OFFV = (BITS == 8) ? 128.f : (float)Q<BITS>::OFF;
  if (__builtin_expect(s < 1e30f, 1)) {
    const float ns = -OFFV * s;
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = __builtin_fmaf(c[j], s, ns);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = (c[j] - OFFV) * s;
  }
  uint4 r;
  r.x = pack_bf16(c[0], c[1]); r.y = pack_bf16(c[2], c[3]); r.z = pack_bf16(c[4], c[5]); r.w = pack_bf16(c[6], c[7]);
  return r;
}

// The same without the branch for huge scales (s >= 1e30 overflows -OFF*s): for consumers that accumulate in fp32
// and are compared to a tolerance, not bit for bit (the weight-gradient GEMM).
template <int BITS>
__device__ __forceinline__ uint4 dequant8_fast(uint32_t lo, uint32_t hi, int seg, float s) {
  constexpr uint32_t REP = (BITS == 8) ? 0x80808080u : Q<BITS>::CODE_MASK * 0x01010101u;
  uint32_t a, b;
  if (BITS == 8) { a = lo ^ REP; b = hi ^ REP; }
  else { a = (lo >> (seg * BITS)) & REP; b = (hi >> (seg * BITS)) & REP; }
  asm volatile("" : "+v"(a), "+v"(b));                       // see dequant8
  float c[8];
  codes8_to_float<BITS>(a, b, c);
  constexpr float OFFV = (BITS == 8) ? 128.f : (float)Q<BITS>::OFF;
  const float ns = -OFFV * s;
#pragma unroll
  for (int j = 0; j < 8; ++j) c[j] = __builtin_fmaf(c[j], s, ns);
  uint4 r;
  r.x = pack_bf16(c[0], c[1]); r.y = pack_bf16(c[2], c[3]); r.z = pack_bf16(c[4], c[5]); r.w = pack_bf16(c[6], c[7]);
  return r;
}

// e^x to about 2 ulp: v_exp_f32 on x*log2(e) with the rounding error of that product (and the low part of
// log2(e)) applied as a first-order correction.  |x| must stay below 2^127 / log2(e) (about 2.3e38): beyond that
// the product overflows and the correction term becomes inf * 0.
__device__ __forceinline__ float exp_fast(float x) {
  const float L2E = 1.44269502162933349609375f, L2E_LO = 1.925963033500e-08f;
  const float t = x * L2E;
  float r = __builtin_fmaf(x, L2E, -t);
  r = __builtin_fmaf(x, L2E_LO, r);
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(e, r * 0.693147182464599609375f, e);
}

// ---- descriptors as the kernels see them -------------------------------------------------------
struct ChanArgs {           // HYC_MODE_CHANNEL
  const uint32_t* plan;     // [H/8]
  const int32_t* idx;       // [k] outlier channels, ascending
  int k;                    // outlier channels
  int groups_per_row;       // H / G
  int chunk_to_group_shift; // log2(G/8)
  int absmax;               // group scale rule: 0 = bf16(bf16(max - min) / (2^b - 1)), 1 = bf16(bf16(2 max|x|) / (2^b - 1)) (1-bit: max|x|)
};

struct ThrArgs {            // HYC_MODE_THRESHOLD
  float thr;                // already a bf16 value
  const uint16_t* scale;
  int64_t sst, ssc;         // scale strides (token, channel)
  int64_t S;
  const uint16_t* L;        // [S, rank]
  const uint16_t* R;        // [rank, H]
  int rank;
  const int32_t* row_ptr;
  const int32_t* cols;
  const uint16_t* vals;
};

// base[c..c+8) = bf16(sum_r L[s,r] * R[r,c]) accumulated in fp32 in increasing r
__device__ __forceinline__ void base8(const ThrArgs& a, int64_t s, int64_t col, int64_t H, float (&b)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) b[j] = 0.f;
  for (int r = 0; r < a.rank; ++r) {
    const float l = bf_to_f(a.L[s * a.rank + r]);
    const uint4 rr = *reinterpret_cast<const uint4*>(a.R + (int64_t)r * H + col);
    float rv[8];
    unpack8(rr, rv);
#pragma unroll
    for (int j = 0; j < 8; ++j) b[j] = __builtin_fmaf(l, rv[j], b[j]);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) b[j] = bfr(b[j]);
}

}  // namespace hyc
