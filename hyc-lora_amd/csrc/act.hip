// Backward of the elementwise operators with the decompression fused in:
//   SiLU      dx = s*(1 + x - x*s)*g, s = sigmoid(x)          operators/efficient_silu.py:50-51
//   GELU      tanh-form derivative                            operators/efficient_gelu.py:49-62
//   Hadamard  dx1 = g*x2, dx2 = x1*g                          operators/efficient_hadamard.py:62-66
// Every intermediate is rounded to bf16 exactly where the reference's torch expression rounds it (each
// torch op on bf16 tensors computes in fp32 and rounds once; Python scalars enter as fp32).
#include <stdlib.h>
#include "abi_util.hpp"
#include "row_kernels.hpp"

namespace hyc {

constexpr int ACT_MUL = 100;   // dx = g * x_hat (one half of the Hadamard backward)

// ---- math helpers ----------------------------------------------------------------------------------
// round two fp32 values to bf16 with one v_cvt_pk_bf16_f32 and widen them again
__device__ __forceinline__ void bfr2(float& a, float& b) {
  const uint32_t pk = pack_bf16(a, b);
  a = bf_lo(pk);
  b = bf_hi(pk);
}
// 1 / d for finite positive d to about 1 ulp; 0 for d = inf
__device__ __forceinline__ float rcp_pos(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  r = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
  return d < 3.0e38f ? r : 0.f;
}
__device__ __forceinline__ float sigmoid_f(float x) { return rcp_pos(1.0f + exp_fast(-x)); }
// tanh: odd polynomial below 0.05 (where 1 - e^{-2|y|} cancels), (1 - e)/(1 + e) above
__device__ __forceinline__ float tanh_f(float y) {
  const float a = __builtin_fminf(__builtin_fabsf(y), 32.0f);   // tanh(32) is 1 in fp32; keeps e^{-2|y|} away from inf * 0
  const float e = exp_fast(-2.0f * a);
  const float big = (1.0f - e) * rcp_pos(1.0f + e);
  const float y2 = a * a;
  float p = __builtin_fmaf(y2, 0.13333333333f, -0.33333333333f);
  p = __builtin_fmaf(y2 * p, a, a);
  const float t = a < 0.05f ? p : big;
  return __builtin_copysignf(t, y);
}

// two elements at a time: every intermediate is rounded to bf16 where torch rounds it, pairs share the conversion
// the derivative alone (a bf16 value): what the gradient is multiplied with
__device__ __forceinline__ void silu_deriv2(float x0, float x1, float& d0, float& d1);
__device__ __forceinline__ void gelu_tanh_deriv2(float x0, float x1, float& d0, float& d1);
__device__ __forceinline__ void silu_grad2(float x0, float x1, float g0, float g1, float& o0, float& o1) {
  float d0, d1;
  silu_deriv2(x0, x1, d0, d1);
  o0 = d0 * g0;           // the caller's pack8 performs the last rounding
  o1 = d1 * g1;
}
__device__ __forceinline__ void silu_deriv2(float x0, float x1, float& d0, float& d1) {
  float s0 = sigmoid_f(x0), s1 = sigmoid_f(x1);
  bfr2(s0, s1);
  float a0 = x0 + 1.0f, a1 = x1 + 1.0f;
  bfr2(a0, a1);
  float b0 = x0 * s0, b1 = x1 * s1;
  bfr2(b0, b1);
  float c0 = a0 - b0, c1 = a1 - b1;
  bfr2(c0, c1);
  d0 = s0 * c0; d1 = s1 * c1;
  bfr2(d0, d1);
}

__device__ __forceinline__ void gelu_tanh_grad2(float x0, float x1, float g0, float g1, float& o0, float& o1) {
  float d0, d1;
  gelu_tanh_deriv2(x0, x1, d0, d1);
  o0 = d0 * g0;
  o1 = d1 * g1;
}
__device__ __forceinline__ void gelu_tanh_deriv2(float x0, float x1, float& d0, float& d1) {
  const float gamma = 0.7978845608028654f;   // sqrt(2/pi)
  const float kappa = 0.044715f;
  const float kappa3 = (float)(3 * 0.044715);
  float q0 = x0 * x0, q1 = x1 * x1;                      // x**2
  bfr2(q0, q1);
  float c0 = q0 * x0, c1 = q1 * x1;                      // x**3 = bf16(bf16(x*x)*x)
  bfr2(c0, c1);
  float k0 = kappa * c0, k1 = kappa * c1;
  bfr2(k0, k1);
  float s0 = x0 + k0, s1 = x1 + k1;
  bfr2(s0, s1);
  float i0 = gamma * s0, i1 = gamma * s1;
  bfr2(i0, i1);
  float t0 = tanh_f(i0), t1 = tanh_f(i1);
  bfr2(t0, t1);
  float A0 = 1.0f + t0, A1 = 1.0f + t1;
  bfr2(A0, A1);
  float u0 = t0 * t0, u1 = t1 * t1;
  bfr2(u0, u1);
  float B0 = 1.0f - u0, B1 = 1.0f - u1;
  bfr2(B0, B1);
  float C0 = B0 * gamma, C1 = B1 * gamma;
  bfr2(C0, C1);
  float D0 = kappa3 * q0, D1 = kappa3 * q1;
  bfr2(D0, D1);
  float E0 = 1.0f + D0, E1 = 1.0f + D1;
  bfr2(E0, E1);
  float F0 = C0 * E0, F1 = C1 * E1;
  bfr2(F0, F1);
  float G0 = x0 * F0, G1 = x1 * F1;
  bfr2(G0, G1);
  float H0 = A0 + G0, H1 = A1 + G1;
  bfr2(H0, H1);
  d0 = 0.5f * H0; d1 = 0.5f * H1;                        // exact
}

template <int ACT>
__device__ __forceinline__ void act_grad8(const float (&x)[8], const float (&g)[8], float (&o)[8]) {
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    if (ACT == HYC_ACT_SILU) silu_grad2(x[j], x[j + 1], g[j], g[j + 1], o[j], o[j + 1]);
    else if (ACT == HYC_ACT_GELU_TANH) gelu_tanh_grad2(x[j], x[j + 1], g[j], g[j + 1], o[j], o[j + 1]);
    else { o[j] = g[j] * x[j]; o[j + 1] = g[j + 1] * x[j + 1]; }
  }
}

// The derivative is a function of one bf16 value, and the reference rounds every step of it to bf16, so a table
// of it is exact by construction.  LUT_EXP binades from 2^LUT_LOG_LO up, both signs; smaller magnitudes (zero
// included) share the first entry (the derivative is the constant 0.5 there), larger ones are computed.
constexpr int LUT_LOG_LO = -12, LUT_EXP = 20;
constexpr uint32_t LUT_LO = (uint32_t)(127 + LUT_LOG_LO) << 7;
constexpr uint32_t LUT_N = LUT_EXP * 128;              // entries per sign
constexpr uint32_t LUT_NEG = 4096;                     // first entry of the negative half
static_assert(LUT_N <= LUT_NEG, "the sign bit is or-ed into the index");

// The table costs a workgroup 2 LUT_N evaluations and saves most of one per element (16 per thread and row), so it
// wants rows x threads of a workgroup above a threshold: measured on 4096-row inputs, 512 pays for the activation
// backward (H = 4096: SiLU 23.8 -> 21.7 us, GELU 40.6 -> 32.9) but not for the forward and gated kernels, whose direct
// evaluation is cheaper next to their other work (they start at 1024, i.e. at 8192 rows of 4096 channels).
// Workgroups of the row kernels whose loop takes one row per iteration: `cap` resident ones, or one per `rows_each`
// rows when that is more.  The kernels without a derivative table (nothing to amortise per workgroup) run faster on
// short loops that the dispatcher balances: measured on 4096 x 11008 / 16 384 x 11008, INT4: activation forward + save
// 44.1 -> 39.3 / 179 -> 161 us at four rows each, product forward + two saves 60.0 -> 54.7 / 291 -> 232 us at two,
// product backward 245 -> 226 us at four (the table kernels lose: gated backward 65 -> 84 us at two rows each).
static int row_loop_grid(int64_t M, int64_t cap, int rows_each) {
  int64_t g = M / rows_each;
  if (g < cap) g = cap;
  if (g > M) g = M;
  return (int)g;
}
// A row of the gated kernels that is too long for one workgroup (their per-thread state caps the workgroup at `most`
// threads) is shared by 2 to 4 workgroups, each a whole number of scale groups (lpg chunks).  Returns the number of
// workgroups per row, 0 if none fits.
static int gated_row_parts(int cps, int most, int lpg) {
  if (cps <= most) return 1;
  for (int n = 2; n <= 4; ++n)
    if (cps % n == 0 && (cps / n) % lpg == 0 && ((cps / n + 63) / 64) * 64 <= most) return n;
  return 0;
}

// the packed code word of a row chunk: written once, read again only in the backward pass
__device__ __forceinline__ void store_codes(uint8_t* p, uint32_t lo, uint32_t hi) {
  const u32x2_t t = {lo, hi};
  __builtin_nontemporal_store(t, reinterpret_cast<u32x2_t*>(p));
}

static inline int lut_pays(int64_t M, int grid, int threads, int64_t least) {
  const int64_t rows_per_wg = (M + grid - 1) / grid;
  return rows_per_wg * threads >= least;
}
constexpr int64_t LUT_PAYS_BWD = 400, LUT_PAYS_OTHER = 1024;

template <int ACT>
__device__ __forceinline__ void lut_fill(uint16_t* lut) {
  for (uint32_t i = 2 * threadIdx.x; i < 2 * LUT_N; i += 2 * blockDim.x) {
    const uint32_t neg = i >= LUT_N ? 1u : 0u, u = i - neg * LUT_N;
    const float x0 = __uint_as_float(((neg << 15) | (LUT_LO + u)) << 16), x1 = __uint_as_float(((neg << 15) | (LUT_LO + u + 1)) << 16);
    float d0, d1;
    if (ACT == HYC_ACT_SILU) silu_deriv2(x0, x1, d0, d1); else gelu_tanh_deriv2(x0, x1, d0, d1);
    lut[neg * LUT_NEG + u] = (uint16_t)(__float_as_uint(d0) >> 16);
    lut[neg * LUT_NEG + u + 1] = (uint16_t)(__float_as_uint(d1) >> 16);
  }
}
// dx of one chunk through the table; false (nothing written) if a lane of the wave holds a value beyond the table
__device__ __forceinline__ bool lut_grad8(const uint16_t* lut, const uint4& xr, const float (&g)[8], float (&o)[8]) {
  const uint32_t w[4] = {xr.x, xr.y, xr.z, xr.w};
  uint32_t idx[8], worst = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t e0 = w[j] & 0x7FFFu, e1 = (w[j] >> 16) & 0x7FFFu;
    const uint32_t u0 = e0 > LUT_LO ? e0 - LUT_LO : 0u, u1 = e1 > LUT_LO ? e1 - LUT_LO : 0u;
    worst = worst > u0 ? worst : u0;
    worst = worst > u1 ? worst : u1;
    idx[2 * j] = ((w[j] >> 3) & LUT_NEG) | u0;
    idx[2 * j + 1] = ((w[j] >> 19) & LUT_NEG) | u1;
  }
  if (__builtin_amdgcn_ballot_w64(worst >= LUT_N) != 0) return false;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = __uint_as_float((uint32_t)lut[idx[j]] << 16) * g[j];
  return true;
}

// fast path: channel source, every lane owns one chunk per segment, next row requested ahead
template <int BITS, int ACT, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_act_bwd_fast(const uint16_t* __restrict__ g, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
               const uint16_t* __restrict__ scales, int64_t M, int64_t H, int CPS, ChanArgs ca,
               uint16_t* __restrict__ dx, int use_lut) {
  constexpr int NSEG = Q<BITS>::NSEG;
  constexpr bool HAS_LUT = ACT == HYC_ACT_SILU || ACT == HYC_ACT_GELU_TANH;
  __shared__ uint16_t lut[HAS_LUT ? LUT_NEG + LUT_N : 1];
  if (HAS_LUT && use_lut) {
    lut_fill<ACT>(lut);
    __syncthreads();
  }
  const int c = threadIdx.x;
  if (c >= CPS) return;                                 // tail of the last wave
  const int64_t SEG = (int64_t)CPS * 8;
  const int seg_groups = CPS >> ca.chunk_to_group_shift;
  uint32_t plan[NSEG];
#pragma unroll
  for (int i = 0; i < NSEG; ++i) plan[i] = ca.plan[i * CPS + c];
  ChunkOutliers<NSEG> co;
  co.init(plan);
  // Every memory instruction of the row loop is an unconditional buffer operation: a row past the end gets a resource
  // of zero bytes (loads return zeros, stores are dropped), an outlier slot the chunk does not have gets an offset
  // beyond every resource.  No branch surrounds a load, so the compiler's waits are sized for the steady state.
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint32_t row_b = 2u * (uint32_t)H, seg_b = 2u * (uint32_t)SEG, gpr_b = 2u * (uint32_t)ca.groups_per_row;
  const uint32_t val_b = 2u * (uint32_t)ca.k;
  const uint32_t xo = 16u * (uint32_t)c, so = 8u * (uint32_t)c;
  uint32_t sco[NSEG], vo0[NSEG], vo1[NSEG];
#pragma unroll
  for (int i = 0; i < NSEG; ++i) {
    sco[i] = 2u * (uint32_t)((c >> ca.chunk_to_group_shift) + i * seg_groups);
    vo0[i] = co.has0[i] ? co.vb[i] : NOWHERE;
    vo1[i] = co.has1[i] ? co.vb[i] + 2u : NOWHERE;
  }
  auto row_of = [&](const void* base, int64_t r, uint32_t bytes) __attribute__((always_inline)) {
    return make_rsrc(static_cast<const char*>(base) + r * (int64_t)bytes, r < M ? bytes : 0u);
  };
  uint2 pk;
  uint4 graw[NSEG];
  uint32_t sc[NSEG], o0[NSEG], o1[NSEG];
  auto request = [&](int64_t r, uint2& pk_, uint4 (&g_)[NSEG], uint32_t (&sc_)[NSEG], uint32_t (&o0_)[NSEG],
                     uint32_t (&o1_)[NSEG]) __attribute__((always_inline)) {
    const BufferRsrc rs_g = row_of(g, r, row_b), rs_s = row_of(stored, r, (uint32_t)SEG);
    const BufferRsrc rs_c = row_of(scales, r, gpr_b), rs_v = row_of(vals, r, val_b);
    pk_ = load_b64(rs_s, so);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      g_[i] = load_b128(rs_g, xo + (uint32_t)i * seg_b);
      sc_[i] = load_b16(rs_c, sco[i]);
      o0_[i] = load_b16(rs_v, vo0[i]);
      o1_[i] = load_b16(rs_v, vo1[i]);
    }
  };
  request(row, pk, graw, sc, o0, o1);
  const int64_t steps = row < M ? (M - row + stride - 1) / stride : 0;
  for (int64_t step = 0; step < steps; ++step, row += stride) {
    uint2 pk_n;
    uint4 g_n[NSEG];
    uint32_t sc_n[NSEG], o0_n[NSEG], o1_n[NSEG];
    request(row + stride, pk_n, g_n, sc_n, o0_n, o1_n);
    const BufferRsrc rs_o = row_of(dx, row, row_b);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float xv[8], gv[8], o[8];
      const float sf = bf_to_f((uint16_t)sc[i]);
      uint4 r = co.splice(i, dequant8<BITS>(pk.x, pk.y, i, sf), o0[i], o1[i], sf);
      if (co.more_pairs) r = splice_more(r, co.more_pairs, ca.plan[i * CPS + c], vals + row * ca.k, true, sf);
      unpack8(graw[i], gv);
      if (!(HAS_LUT && use_lut && lut_grad8(lut, r, gv, o))) {
        unpack8(r, xv);
        act_grad8<ACT>(xv, gv, o);
      }
      store_b128_stream(rs_o, xo + (uint32_t)i * seg_b, pack8(o));
    }
    pk = pk_n;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) { graw[i] = g_n[i]; sc[i] = sc_n[i]; o0[i] = o0_n[i]; o1[i] = o1_n[i]; }
  }
}

// Hadamard backward in one pass when both operands are channel-compressed with the same code width (the thread to
// chunk mapping then agrees): g is read once, dx1 = g * x2_hat, dx2 = x1_hat * g.
template <int BITS, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_hadamard_bwd_fast(const uint16_t* __restrict__ g, const uint8_t* __restrict__ st1, const uint16_t* __restrict__ v1,
                    const uint16_t* __restrict__ s1, ChanArgs c1, const uint8_t* __restrict__ st2,
                    const uint16_t* __restrict__ v2, const uint16_t* __restrict__ s2, ChanArgs c2, int64_t M, int64_t H,
                    int CPS, uint16_t* __restrict__ dx1, uint16_t* __restrict__ dx2) {
  constexpr int NSEG = Q<BITS>::NSEG;
  const int c = threadIdx.x;
  if (c >= CPS) return;                                 // tail of the last wave
  const int64_t SEG = (int64_t)CPS * 8;
  const int sg1 = CPS >> c1.chunk_to_group_shift, sg2 = CPS >> c2.chunk_to_group_shift;
  ChunkOutliers<NSEG> o1, o2;
  {
    uint32_t p1[NSEG], p2[NSEG];
#pragma unroll
    for (int i = 0; i < NSEG; ++i) { p1[i] = c1.plan[i * CPS + c]; p2[i] = c2.plan[i * CPS + c]; }
    o1.init(p1);
    o2.init(p2);
  }
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint16_t* gp = g + row * H + 8 * c;
  uint16_t* d1p = dx1 + row * H + 8 * c;
  uint16_t* d2p = dx2 + row * H + 8 * c;
  const uint8_t* sp1 = st1 + row * SEG + 8 * c;
  const uint8_t* sp2 = st2 + row * SEG + 8 * c;
  const uint16_t* vp1 = v1 + row * c1.k;
  const uint16_t* vp2 = v2 + row * c2.k;
  const uint16_t* scp1 = s1 + row * c1.groups_per_row + (c >> c1.chunk_to_group_shift);
  const uint16_t* scp2 = s2 + row * c2.groups_per_row + (c >> c2.chunk_to_group_shift);
  const int64_t xstep = stride * H, sstep = stride * SEG;
  uint2 pk1 = make_uint2(0, 0), pk2 = make_uint2(0, 0);
  uint4 graw[NSEG];
  uint32_t sc1[NSEG], sc2[NSEG], a0[NSEG], a1[NSEG], b0[NSEG], b1[NSEG];
  if (row < M) {
    pk1 = *reinterpret_cast<const uint2*>(sp1);
    pk2 = *reinterpret_cast<const uint2*>(sp2);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      graw[i] = *reinterpret_cast<const uint4*>(gp + i * SEG);
      sc1[i] = scp1[i * sg1]; sc2[i] = scp2[i * sg2];
    }
    o1.request(vp1, a0, a1);
    o2.request(vp2, b0, b1);
  }
  for (; row < M; row += stride) {
    uint2 pk1_n = make_uint2(0, 0), pk2_n = make_uint2(0, 0);
    uint4 g_n[NSEG];
    uint32_t sc1_n[NSEG], sc2_n[NSEG], a0_n[NSEG], a1_n[NSEG], b0_n[NSEG], b1_n[NSEG];
    if (row + stride < M) {
      pk1_n = *reinterpret_cast<const uint2*>(sp1 + sstep);
      pk2_n = *reinterpret_cast<const uint2*>(sp2 + sstep);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        g_n[i] = *reinterpret_cast<const uint4*>(gp + xstep + i * SEG);
        sc1_n[i] = scp1[stride * c1.groups_per_row + i * sg1];
        sc2_n[i] = scp2[stride * c2.groups_per_row + i * sg2];
      }
      o1.request(vp1 + stride * c1.k, a0_n, a1_n);
      o2.request(vp2 + stride * c2.k, b0_n, b1_n);
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float x1[8], x2[8], gv[8], r1[8], r2[8];
      const float f1 = bf_to_f((uint16_t)sc1[i]), f2 = bf_to_f((uint16_t)sc2[i]);
      uint4 q1 = o1.splice(i, dequant8<BITS>(pk1.x, pk1.y, i, f1), a0[i], a1[i], f1);
      uint4 q2 = o2.splice(i, dequant8<BITS>(pk2.x, pk2.y, i, f2), b0[i], b1[i], f2);
      if (o1.more_pairs) q1 = splice_more(q1, o1.more_pairs, c1.plan[i * CPS + c], vp1, true, f1);
      if (o2.more_pairs) q2 = splice_more(q2, o2.more_pairs, c2.plan[i * CPS + c], vp2, true, f2);
      unpack8(q1, x1);
      unpack8(q2, x2);
      unpack8(graw[i], gv);
#pragma unroll
      for (int j = 0; j < 8; ++j) { r1[j] = gv[j] * x2[j]; r2[j] = x1[j] * gv[j]; }
      store_stream(d1p + i * SEG, pack8(r1));
      store_stream(d2p + i * SEG, pack8(r2));
    }
    pk1 = pk1_n; pk2 = pk2_n;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      graw[i] = g_n[i]; sc1[i] = sc1_n[i]; sc2[i] = sc2_n[i];
      a0[i] = a0_n[i]; a1[i] = a1_n[i]; b0[i] = b0_n[i]; b1[i] = b1_n[i];
    }
    gp += xstep; d1p += xstep; d2p += xstep; sp1 += sstep; sp2 += sstep;
    vp1 += stride * c1.k; vp2 += stride * c2.k;
    scp1 += stride * c1.groups_per_row; scp2 += stride * c2.groups_per_row;
  }
}

// One channel-compressed operand of a fast row kernel: the thread's view of it (chunk c of every segment), with the
// current row's codes / scales / outliers in registers; next() reloads them for the following row as soon as the
// current one has been decoded (no second register set).
template <int BITS>
struct ChanSource {
  static constexpr int NSEG = Q<BITS>::NSEG;
  ChunkOutliers<NSEG> co;
  const uint8_t* sp; const uint16_t* vp; const uint16_t* scp; const uint32_t* plan;
  int64_t sstep, vstep, scstep;
  int seg_groups;
  uint2 pk;
  uint32_t sc[NSEG], o0[NSEG], o1[NSEG];

  __device__ __forceinline__ void init(const uint8_t* stored, const uint16_t* vals, const uint16_t* scales, const ChanArgs& a,
                                       int c, int CPS, int64_t row, int64_t stride) {
    uint32_t p[NSEG];
#pragma unroll
    for (int i = 0; i < NSEG; ++i) p[i] = a.plan[i * CPS + c];
    co.init(p);
    plan = a.plan + c;
    seg_groups = CPS >> a.chunk_to_group_shift;
    sp = stored + row * ((int64_t)CPS * 8) + 8 * c;
    vp = vals + row * a.k;
    scp = scales + row * a.groups_per_row + (c >> a.chunk_to_group_shift);
    sstep = stride * (int64_t)CPS * 8; vstep = stride * a.k; scstep = stride * a.groups_per_row;
    pk = make_uint2(0, 0);
  }
  __device__ __forceinline__ void request_first() {
    pk = *reinterpret_cast<const uint2*>(sp);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) sc[i] = scp[i * seg_groups];
    co.request(vp, o0, o1);
  }
  __device__ __forceinline__ void next() {
    sp += sstep; vp += vstep; scp += scstep;
    request_first();
  }
  __device__ __forceinline__ void decode(int i, int CPS, float (&x)[8]) const {
    const float f = bf_to_f((uint16_t)sc[i]);
    uint4 q = co.splice(i, dequant8<BITS>(pk.x, pk.y, i, f), o0[i], o1[i], f);
    if (co.more_pairs) q = splice_more(q, co.more_pairs, plan[i * CPS], vp, true, f);
    unpack8(q, x);
  }
};

// Backward of h = act(gate) * up in one pass, with the three saved activations the separate operators keep:
// a_hat = decompress(act(gate)), up_hat, gate_hat.  d_up = a_hat * g;  d_gate = act'(gate_hat) * bf16(g * up_hat) -
// the same roundings as hyc_hadamard_bwd followed by hyc_act_bwd, without the round trip of g * up_hat through memory.
template <int BITS, int ACT, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_gated_act_bwd_fast(const uint16_t* __restrict__ g, const uint8_t* __restrict__ st_a, const uint16_t* __restrict__ v_a,
                     const uint16_t* __restrict__ s_a, ChanArgs c_a, const uint8_t* __restrict__ st_u,
                     const uint16_t* __restrict__ v_u, const uint16_t* __restrict__ s_u, ChanArgs c_u,
                     const uint8_t* __restrict__ st_g, const uint16_t* __restrict__ v_g, const uint16_t* __restrict__ s_g,
                     ChanArgs c_g, int64_t M, int64_t H, int CPS, int cps_wg, uint16_t* __restrict__ d_gate,
                     uint16_t* __restrict__ d_up, int use_lut) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ uint16_t lut[LUT_NEG + LUT_N];             // the activation's derivative, see lut_fill
  if (use_lut) {
    lut_fill<ACT>(lut);
    __syncthreads();
  }
  // (a row too long for one workgroup's registers is shared by gridDim.y workgroups of cps_wg chunks each, a whole
  // number of scale groups: nothing in this kernel looks beyond a scale group)
  const int c = (int)blockIdx.y * cps_wg + (int)threadIdx.x;
  if ((int)threadIdx.x >= cps_wg) return;               // tail of the last wave
  const int64_t SEG = (int64_t)CPS * 8;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  ChanSource<BITS> A, U, G;
  A.init(st_a, v_a, s_a, c_a, c, CPS, row, stride);
  U.init(st_u, v_u, s_u, c_u, c, CPS, row, stride);
  G.init(st_g, v_g, s_g, c_g, c, CPS, row, stride);
  const uint16_t* gp = g + row * H + 8 * c;
  uint16_t* dgp = d_gate + row * H + 8 * c;
  uint16_t* dup = d_up + row * H + 8 * c;
  const int64_t xstep = stride * H;
  uint4 graw[NSEG];
  if (row < M) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) graw[i] = *reinterpret_cast<const uint4*>(gp + i * SEG);
    A.request_first(); U.request_first(); G.request_first();
  }
  for (; row < M; row += stride) {
    uint4 g_n[NSEG];
    const bool more = row + stride < M;
    if (more) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) g_n[i] = *reinterpret_cast<const uint4*>(gp + xstep + i * SEG);
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float xa[8], xu[8], xg[8], gv[8], t[8], r[8];
      A.decode(i, CPS, xa);
      U.decode(i, CPS, xu);
      G.decode(i, CPS, xg);
      if (i == NSEG - 1 && more) { A.next(); U.next(); G.next(); }   // the compressed rows are decoded: reload
      unpack8(graw[i], gv);
#pragma unroll
      for (int j = 0; j < 8; ++j) { r[j] = xa[j] * gv[j]; t[j] = gv[j] * xu[j]; }
      store_stream(dup + i * SEG, pack8(r));
      unpack8(pack8(t), t);                             // the gradient of act(gate), rounded to bf16 as a tensor would be
      if (!(use_lut && lut_grad8(lut, pack8(xg), t, r))) act_grad8<ACT>(xg, t, r);
      store_stream(dgp + i * SEG, pack8(r));
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) graw[i] = g_n[i];
    gp += xstep; dgp += xstep; dup += xstep;
  }
}

// ---- forward of h = act(gate) * up with the three saves fused in ----------------------------------------------
// The activation value as the framework computes it for a bf16 tensor: fp32 arithmetic with the accurate library
// exp / erf, one rounding to bf16 (operators/efficient_silu.py:16 F.silu, operators/efficient_gelu.py:16 F.gelu).
// SiLU takes a short cut that cannot change the bf16 result: x * rcp(1 + exp(-x)) with the hardware exp and a refined
// reciprocal is within a few fp32 ulp of the library expression; only when that value lies within 32 ulp of a bf16
// rounding boundary (1 element in 1000), or where the short cut loses accuracy (|x| >= 80, tiny results), is the
// library expression evaluated.  Both forms then round to the same bf16 value for every input (tested on all 65 536).
template <int ACT>
__device__ __forceinline__ float act_value(float x) {
  if (ACT == HYC_ACT_SILU) {
    float f = x * rcp_pos(1.0f + exp_fast(-x));
    const uint32_t low = __float_as_uint(f) & 0xFFFFu;            // the bits a bf16 rounding drops
    const bool decided = (low - 0x7FE0u > 0x40u) && __builtin_fabsf(x) < 80.0f && __builtin_fabsf(f) > 1e-30f;
    if (__builtin_expect(!decided, 0)) f = x / (1.0f + expf(-x));
    return f;
  }
  return (x * 0.5f) * (1.0f + erff(x * 0.70710678118654752440f));
}

// The forward value is a function of one bf16 input as well: the same table layout, filled with bf16(act(x)).
// Nothing is shared below the table here (act(x) ~ x/2 near zero): such inputs, zero included, are computed.
template <int ACT>
__device__ __forceinline__ void lut_fill_value(uint16_t* lut) {
  for (uint32_t i = threadIdx.x; i < 2 * LUT_N; i += blockDim.x) {
    const uint32_t neg = i >= LUT_N ? 1u : 0u, u = i - neg * LUT_N;
    lut[neg * LUT_NEG + u] = f_to_bf(act_value<ACT>(__uint_as_float(((neg << 15) | (LUT_LO + u)) << 16)));
  }
}
// bf16(act(x)) of one chunk through the table; false (nothing written) if a lane of the wave holds a value outside it
__device__ __forceinline__ bool lut_value8(const uint16_t* lut, const uint4& xr, uint4& out) {
  const uint32_t w[4] = {xr.x, xr.y, xr.z, xr.w};
  uint32_t idx[8], worst = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t u0 = (w[j] & 0x7FFFu) - LUT_LO, u1 = ((w[j] >> 16) & 0x7FFFu) - LUT_LO;     // wraps below the table
    worst = worst > u0 ? worst : u0;
    worst = worst > u1 ? worst : u1;
    idx[2 * j] = ((w[j] >> 3) & LUT_NEG) | u0;
    idx[2 * j + 1] = ((w[j] >> 19) & LUT_NEG) | u1;
  }
  if (__builtin_amdgcn_ballot_w64(worst >= LUT_N) != 0) return false;
  out.x = (uint32_t)lut[idx[0]] | ((uint32_t)lut[idx[1]] << 16);
  out.y = (uint32_t)lut[idx[2]] | ((uint32_t)lut[idx[3]] << 16);
  out.z = (uint32_t)lut[idx[4]] | ((uint32_t)lut[idx[5]] << 16);
  out.w = (uint32_t)lut[idx[6]] | ((uint32_t)lut[idx[7]] << 16);
  return true;
}

struct GatedFwdSite {       // one compressed output
  ChanArgs ca;
  uint8_t* stored;
  uint16_t* vals;
  uint16_t* scales;
};

// One pass: reads gate and up (row pitches ldg, ldu: they may be column slices of one projection output), writes
// h = bf16(bf16(act(gate)) * up) and the channel-compressed forms of act(gate), up and gate - what F.silu,
// three hyc_compress calls and a multiply write and re-read through memory.  act(gate) itself is never stored.
template <int BITS, int LPGT, int ACT, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_gated_act_fwd_fast(const uint16_t* __restrict__ gate, int64_t ldg, const uint16_t* __restrict__ up, int64_t ldu, int64_t M,
                     int64_t H, int CPS, int cps_wg, GatedFwdSite sa, GatedFwdSite su, GatedFwdSite sg, uint16_t* __restrict__ h,
                     int use_lut) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ uint16_t lut[LUT_NEG + LUT_N];
  if (use_lut) {
    lut_fill_value<ACT>(lut);
    __syncthreads();
  }
  const int c = (int)blockIdx.y * cps_wg + (int)threadIdx.x;    // (gridDim.y workgroups of cps_wg chunks share a long row)
  if ((int)threadIdx.x >= cps_wg) return;               // tail of the last wave; scale groups never straddle it
  const int64_t SEG = (int64_t)CPS * 8;
  const bool leader = (c & (LPGT - 1)) == 0;
  const int shift = sa.ca.chunk_to_group_shift;         // the three sites share the group width
  const int seg_groups = CPS >> shift;
  const int gpr = sa.ca.groups_per_row;
  uint32_t km_a[NSEG][4], km_u[NSEG][4], km_g[NSEG][4];
  {
    uint32_t plan[NSEG];
    ChunkOutliers<NSEG> co;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) plan[i] = sa.ca.plan[i * CPS + c];
    co.init(plan);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km_a[i]);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) plan[i] = su.ca.plan[i * CPS + c];
    co.init(plan);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km_u[i]);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) plan[i] = sg.ca.plan[i * CPS + c];
    co.init(plan);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km_g[i]);
  }
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint16_t* grow = gate + row * ldg;
  const uint16_t* urow = up + row * ldu;
  uint16_t* hp = h + row * H + 8 * c;
  const int64_t gstep = stride * ldg, ustep = stride * ldu, hstep = stride * H, sstep = stride * SEG, scstep = stride * gpr;
  int64_t soff = row * SEG + 8 * c, scoff = row * gpr + (c >> shift);
  // outlier channels, kept verbatim: thread c copies channel idx[c] of each site (+ CPS, ... when a site has more of
  // them than the row has threads); the index is read once, the element at the top of the row's iteration
  const bool ga = c < sa.ca.k, gu = c < su.ca.k, gg = c < sg.ca.k;
  const int ia = ga ? sa.ca.idx[c] : 0, iu = gu ? su.ca.idx[c] : 0, ig = gg ? sg.ca.idx[c] : 0;
  uint16_t oa = 0, ou = 0, og = 0;
  uint4 graw[NSEG], uraw[NSEG];
  if (row < M) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      graw[i] = *reinterpret_cast<const uint4*>(grow + i * SEG + 8 * c);
      uraw[i] = *reinterpret_cast<const uint4*>(urow + i * SEG + 8 * c);
    }
  }
  for (; row < M; row += stride) {
    // (by every lane, and ahead of the next row's requests: a branch around a load ends in a full wait, and loads
    // return in order, so the wait for these at the end of the row leaves the next row's in flight)
    oa = grow[ia]; ou = urow[iu]; og = grow[ig];
    uint4 g_n[NSEG], u_n[NSEG];
    if (row + stride < M) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        g_n[i] = *reinterpret_cast<const uint4*>(grow + gstep + i * SEG + 8 * c);
        u_n[i] = *reinterpret_cast<const uint4*>(urow + ustep + i * SEG + 8 * c);
      }
    }
    uint32_t lo_a = 0, hi_a = 0, lo_u = 0, hi_u = 0, lo_g = 0, hi_g = 0;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float gv[8], uv[8], av[8], v[8];
      unpack8(uraw[i], uv);
      uint4 araw;                                       // act(gate) as the bf16 tensor the framework would hold
      if (!(use_lut && lut_value8(lut, graw[i], araw))) {
        unpack8(graw[i], gv);
#pragma unroll
        for (int j = 0; j < 8; ++j) av[j] = act_value<ACT>(gv[j]);
        araw = pack8(av);
      }
      unpack8(araw, av);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = av[j] * uv[j];
      store_stream(hp + i * SEG, pack8(v));
      uint32_t cl, ch;
      unpack8(make_uint4(araw.x & km_a[i][0], araw.y & km_a[i][1], araw.z & km_a[i][2], araw.w & km_a[i][3]), v);
      float s = quant_seg<BITS, LPGT>(v, LPGT, cl, ch, sa.ca.absmax != 0);
      if (leader) sa.scales[scoff + i * seg_groups] = f_to_bf(s);
      if (BITS == 8) { lo_a = cl; hi_a = ch; } else { lo_a |= cl << (i * BITS); hi_a |= ch << (i * BITS); }
      unpack8(make_uint4(uraw[i].x & km_u[i][0], uraw[i].y & km_u[i][1], uraw[i].z & km_u[i][2], uraw[i].w & km_u[i][3]), v);
      s = quant_seg<BITS, LPGT>(v, LPGT, cl, ch, su.ca.absmax != 0);
      if (leader) su.scales[scoff + i * seg_groups] = f_to_bf(s);
      if (BITS == 8) { lo_u = cl; hi_u = ch; } else { lo_u |= cl << (i * BITS); hi_u |= ch << (i * BITS); }
      unpack8(make_uint4(graw[i].x & km_g[i][0], graw[i].y & km_g[i][1], graw[i].z & km_g[i][2], graw[i].w & km_g[i][3]), v);
      s = quant_seg<BITS, LPGT>(v, LPGT, cl, ch, sg.ca.absmax != 0);
      if (leader) sg.scales[scoff + i * seg_groups] = f_to_bf(s);
      if (BITS == 8) { lo_g = cl; hi_g = ch; } else { lo_g |= cl << (i * BITS); hi_g |= ch << (i * BITS); }
    }
    store_codes(sa.stored + soff, lo_a, hi_a);
    store_codes(su.stored + soff, lo_u, hi_u);
    store_codes(sg.stored + soff, lo_g, hi_g);
    if (ga) {
      sa.vals[row * sa.ca.k + c] = f_to_bf(act_value<ACT>(bf_to_f(oa)));
      for (int t = c + CPS; t < sa.ca.k; t += CPS)
        sa.vals[row * sa.ca.k + t] = f_to_bf(act_value<ACT>(bf_to_f(grow[sa.ca.idx[t]])));
    }
    if (gu) {
      su.vals[row * su.ca.k + c] = ou;
      for (int t = c + CPS; t < su.ca.k; t += CPS) su.vals[row * su.ca.k + t] = urow[su.ca.idx[t]];
    }
    if (gg) {
      sg.vals[row * sg.ca.k + c] = og;
      for (int t = c + CPS; t < sg.ca.k; t += CPS) sg.vals[row * sg.ca.k + t] = grow[sg.ca.idx[t]];
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) { graw[i] = g_n[i]; uraw[i] = u_n[i]; }
    grow += gstep; urow += ustep; hp += hstep; soff += sstep; scoff += scstep;
  }
}

// The same idea for the operators taken one at a time (what a module swap installs): NIN = 1: y = act(x) and the
// compressed x (EfficientMemorySiLU / GELU forward, efficient_silu.py:13-40, efficient_gelu.py:13-40);
// NIN = 2: y = x1 * x2 and both operands compressed (EfficientMemoryHadamard forward, efficient_hadamard.py:11-53).
// Every operand is read once.
template <int BITS, int LPGT, int ACT, int NIN, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_ew_fwd_fast(const uint16_t* __restrict__ x1, int64_t ld1, const uint16_t* __restrict__ x2, int64_t ld2, int64_t M, int64_t H,
              int CPS, GatedFwdSite s1, GatedFwdSite s2, uint16_t* __restrict__ y, int use_lut) {
  constexpr int NSEG = Q<BITS>::NSEG;
  constexpr bool HAS_LUT = NIN == 1;
  __shared__ uint16_t lut[HAS_LUT ? LUT_NEG + LUT_N : 1];
  if (HAS_LUT && use_lut) {
    lut_fill_value<ACT == ACT_MUL ? HYC_ACT_SILU : ACT>(lut);
    __syncthreads();
  }
  const int c = threadIdx.x;
  if (c >= CPS) return;                                 // tail of the last wave; scale groups never straddle it
  const int64_t SEG = (int64_t)CPS * 8;
  const bool leader = (c & (LPGT - 1)) == 0;
  const int shift = s1.ca.chunk_to_group_shift;
  const int seg_groups = CPS >> shift;
  const int gpr = s1.ca.groups_per_row;
  uint32_t km[NIN][NSEG][4];
  {
    uint32_t plan[NSEG];
    ChunkOutliers<NSEG> co;
#pragma unroll
    for (int n = 0; n < NIN; ++n) {
      const ChanArgs& ca = n == 0 ? s1.ca : s2.ca;
#pragma unroll
      for (int i = 0; i < NSEG; ++i) plan[i] = ca.plan[i * CPS + c];
      co.init(plan);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km[n][i]);
    }
  }
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint16_t* r1 = x1 + row * ld1;
  const uint16_t* r2 = NIN == 2 ? x2 + row * ld2 : nullptr;
  uint16_t* yp = y + row * H + 8 * c;
  const int64_t step1 = stride * ld1, step2 = stride * ld2, ystep = stride * H, sstep = stride * SEG, scstep = stride * gpr;
  int64_t soff = row * SEG + 8 * c, scoff = row * gpr + (c >> shift);
  // outlier channels, kept verbatim: thread c copies channel idx[c] of each operand (+ CPS, ... when there are more of
  // them than the row has threads); the index is read once, the element at the top of the row's iteration
  const bool g1 = c < s1.ca.k, g2 = NIN == 2 && c < s2.ca.k;
  const int i1 = g1 ? s1.ca.idx[c] : 0, i2 = g2 ? s2.ca.idx[c] : 0;
  uint16_t ov1 = 0, ov2 = 0;
  uint4 raw[NIN][NSEG];
  if (row < M) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      raw[0][i] = *reinterpret_cast<const uint4*>(r1 + i * SEG + 8 * c);
      if (NIN == 2) raw[NIN - 1][i] = *reinterpret_cast<const uint4*>(r2 + i * SEG + 8 * c);
    }
  }
  for (; row < M; row += stride) {
    // (by every lane, and ahead of the next row's requests: a branch around a load ends in a full wait, and loads
    // return in order, so the wait for these at the end of the row leaves the next row's in flight)
    ov1 = r1[i1];
    if (NIN == 2) ov2 = r2[i2];
    uint4 nxt[NIN][NSEG];
    if (row + stride < M) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        nxt[0][i] = *reinterpret_cast<const uint4*>(r1 + step1 + i * SEG + 8 * c);
        if (NIN == 2) nxt[NIN - 1][i] = *reinterpret_cast<const uint4*>(r2 + step2 + i * SEG + 8 * c);
      }
    }
    uint32_t lo[NIN], hi[NIN];
#pragma unroll
    for (int n = 0; n < NIN; ++n) { lo[n] = 0; hi[n] = 0; }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float a[8], v[8];
      uint4 yraw;
      if (NIN == 2) {
        unpack8(raw[0][i], a);
        unpack8(raw[NIN - 1][i], v);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = a[j] * v[j];
        yraw = pack8(v);
      } else if (!(use_lut && lut_value8(lut, raw[0][i], yraw))) {
        unpack8(raw[0][i], a);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = act_value<ACT>(a[j]);
        yraw = pack8(v);
      }
      store_stream(yp + i * SEG, yraw);
#pragma unroll
      for (int n = 0; n < NIN; ++n) {
        const uint4 r = raw[n][i];
        unpack8(make_uint4(r.x & km[n][i][0], r.y & km[n][i][1], r.z & km[n][i][2], r.w & km[n][i][3]), v);
        uint32_t cl, ch;
        const float s = quant_seg<BITS, LPGT>(v, LPGT, cl, ch, (n == 0 ? s1.ca.absmax : s2.ca.absmax) != 0);
        if (leader) (n == 0 ? s1.scales : s2.scales)[scoff + i * seg_groups] = f_to_bf(s);
        if (BITS == 8) { lo[n] = cl; hi[n] = ch; } else { lo[n] |= cl << (i * BITS); hi[n] |= ch << (i * BITS); }
      }
    }
    store_codes(s1.stored + soff, lo[0], hi[0]);
    if (NIN == 2) store_codes(s2.stored + soff, lo[NIN - 1], hi[NIN - 1]);
    if (g1) {
      s1.vals[row * s1.ca.k + c] = ov1;
      for (int t = c + CPS; t < s1.ca.k; t += CPS) s1.vals[row * s1.ca.k + t] = r1[s1.ca.idx[t]];
    }
    if (g2) {
      s2.vals[row * s2.ca.k + c] = ov2;
      for (int t = c + CPS; t < s2.ca.k; t += CPS) s2.vals[row * s2.ca.k + t] = r2[s2.ca.idx[t]];
    }
#pragma unroll
    for (int n = 0; n < NIN; ++n)
#pragma unroll
      for (int i = 0; i < NSEG; ++i) raw[n][i] = nxt[n][i];
    r1 += step1; if (NIN == 2) r2 += step2;
    yp += ystep; soff += sstep; scoff += scstep;
  }
}

// SRC 0 = channel-compressed, 2 = dense bf16
template <int BITS, int SRC, int ACT>
__global__ void __launch_bounds__(1024)
k_act_bwd(const uint16_t* __restrict__ g, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
          const uint16_t* __restrict__ scales, int64_t M, int64_t H, int CPS, int iters, ChanArgs ca,
          uint16_t* __restrict__ dx, int use_lut) {
  constexpr int NSEG = Q<BITS>::NSEG;
  constexpr bool HAS_LUT = ACT == HYC_ACT_SILU || ACT == HYC_ACT_GELU_TANH;
  __shared__ uint16_t lut[HAS_LUT ? LUT_NEG + LUT_N : 1];   // the derivative table of the fast kernel
  if (HAS_LUT && use_lut) {
    lut_fill<ACT>(lut);
    __syncthreads();
  }
  const int64_t SEG = (int64_t)CPS * 8;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    for (int it = 0; it < iters; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
        uint2 pk = make_uint2(0, 0);
        if (SRC == 0) pk = *reinterpret_cast<const uint2*>(stored + row * SEG + 8 * c);
        uint4 graw[NSEG];
#pragma unroll
        for (int i = 0; i < NSEG; ++i) graw[i] = *reinterpret_cast<const uint4*>(g + row * H + i * SEG + 8 * c);
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          const int64_t col = i * SEG + 8 * c;
          float xv[8], gv[8], o[8];
          uint4 xr;
          if (SRC == 0) {
            decode_chan<BITS>(pk.x, pk.y, i, c, CPS, ca, vals + row * ca.k, scales + row * ca.groups_per_row, xv);
            if (HAS_LUT) xr = pack8(xv);
          } else {
            xr = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(stored) + row * H + col);
            unpack8(xr, xv);
          }
          unpack8(graw[i], gv);
          if (!(HAS_LUT && use_lut && lut_grad8(lut, xr, gv, o))) act_grad8<ACT>(xv, gv, o);
          store_stream(dx + row * H + col, pack8(o));
        }
      }
    }
  }
}

template <int ACT>
static int launch_act(const void* g, const void* stored, const void* vals, const void* scales, int64_t M, int64_t H,
                      const hyc_desc* d, void* dx, void* stream, const char* who) {
  if (!d) return fail(HYC_EFAULT, "%s: null descriptor", who);
  if (M < 0) return fail(HYC_EINVAL, "%s: M=%lld", who, (long long)M);
  if (d->mode == HYC_MODE_THRESHOLD)
    return fail(HYC_ENOTSUP, "%s: threshold-mode activations are decompressed first (hyc_decompress) and passed with HYC_MODE_DENSE", who);
  if (d->mode != HYC_MODE_CHANNEL && d->mode != HYC_MODE_DENSE) return fail(HYC_EINVAL, "%s: mode=%d", who, d->mode);
  RowGeom geo;
  int rc = row_geom(H, d->bits, &geo);
  if (rc) return rc;
  ChanArgs ca = {}; int lpg = 16;
  if (d->mode == HYC_MODE_CHANNEL && (rc = make_chan_args(d, geo, &ca, &lpg))) return rc;
  if (M == 0) return HYC_OK;
  if (!g || !stored || !dx) return fail(HYC_EFAULT, "%s: null buffer", who);
  if (d->mode == HYC_MODE_CHANNEL && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "%s: null vals/scales", who);
  if (!aligned16(g) || !aligned16(dx) || !aligned8(stored) || (d->mode == HYC_MODE_DENSE && !aligned16(stored)))
    return fail(HYC_EINVAL, "%s: g, dx must be 16-byte aligned, stored 8-byte (16 when dense)", who);
  const int64_t cap = 256 * (geo.threads >= 512 ? 3 : 8);
  int grid = (int)(M < cap ? M : cap);
  // Every workgroup of the activation kernels fills its own derivative table, so workgroups of four waves or fewer get
  // more rows each instead of the chip more workgroups: about two waves per SIMD (4096 x 4096 INT2, 128 threads, 2048
  // -> 1024 workgroups: GELU 40 -> 25 us, SiLU 25 -> 19 us; INT4, 256 threads, 2048 -> 512: GELU 27.6 -> 17.3 us, SiLU
  // 17.6 -> 15.2 us, and 232 -> 221 us at 65 536 rows; H = 5120, 320 threads, 2048 -> 768: 36.0 -> 21.2 / 24.6 -> 18.6 us)
  // Rows of eight waves or more (one workgroup per CU at a time): about eight rows per workgroup, in whole rounds of the
  // 256 CUs (2048 x 11008: GELU 24.5 -> 20.5 us, 4096 rows: 38.9 -> 37.5, 16 384 rows: SiLU 160.7 -> 152.3).
  if (ACT != ACT_MUL && geo.iters == 1) {
    int fewer = geo.threads <= 128 ? 1024 : geo.threads <= 256 ? 512 : 768;
    if (geo.threads >= 512) {
      const int64_t by_rows = (M / 8 / 256) * 256;
      fewer = (int)(by_rows < 256 ? 256 : by_rows > 2048 ? 2048 : by_rows);
      grid = (int)(M < fewer ? M : fewer);
    }
    if (grid > fewer) grid = fewer;
  }
  hipStream_t st = begin_launch(stream);
  const int use_lut = lut_pays(M, grid, geo.threads * geo.iters, LUT_PAYS_BWD);
  if (d->mode == HYC_MODE_CHANNEL && geo.iters == 1 && d->bits != 1) {
#define HYC_ACT_FAST(B_)                                                                                       \
  do {                                                                                                         \
    if (geo.threads <= 256)                                                                                    \
      hipLaunchKernelGGL((k_act_bwd_fast<B_, ACT, 256>), dim3(grid), dim3(geo.threads), 0, st,                 \
                         static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored),                 \
                         static_cast<const uint16_t*>(vals), static_cast<const uint16_t*>(scales), M, H, geo.cps, ca, \
                         static_cast<uint16_t*>(dx), use_lut);                                                 \
    else                                                                                                       \
      hipLaunchKernelGGL((k_act_bwd_fast<B_, ACT, 1024>), dim3(grid), dim3(geo.threads), 0, st,                \
                         static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored),                 \
                         static_cast<const uint16_t*>(vals), static_cast<const uint16_t*>(scales), M, H, geo.cps, ca, \
                         static_cast<uint16_t*>(dx), use_lut);                                                 \
  } while (0)
    if (d->bits == 2) HYC_ACT_FAST(2);
    else if (d->bits == 4) HYC_ACT_FAST(4);
    else HYC_ACT_FAST(8);
#undef HYC_ACT_FAST
    return check_launch(who);
  }
#define HYC_ACT_LAUNCH(B_, S_)                                                                            \
  hipLaunchKernelGGL((k_act_bwd<B_, S_, ACT>), dim3(grid), dim3(geo.threads), 0, st,                      \
                     static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored),                \
                     static_cast<const uint16_t*>(vals), static_cast<const uint16_t*>(scales), M, H, geo.cps, \
                     geo.iters, ca, static_cast<uint16_t*>(dx), use_lut)
  if (d->mode == HYC_MODE_CHANNEL) {
    switch (d->bits) {
      case 1: HYC_ACT_LAUNCH(1, 0); break;
      case 2: HYC_ACT_LAUNCH(2, 0); break;
      case 4: HYC_ACT_LAUNCH(4, 0); break;
      default: HYC_ACT_LAUNCH(8, 0); break;
    }
  } else {
    switch (d->bits) {
      case 1: HYC_ACT_LAUNCH(1, 2); break;
      case 2: HYC_ACT_LAUNCH(2, 2); break;
      case 4: HYC_ACT_LAUNCH(4, 2); break;
      default: HYC_ACT_LAUNCH(8, 2); break;
    }
  }
#undef HYC_ACT_LAUNCH
  return check_launch(who);
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_act_bwd(int32_t act, const void* g, const void* stored, const void* vals, const void* scales, int64_t M,
                int64_t H, const hyc_desc* d, void* dx, void* stream) {
  if (act == HYC_ACT_SILU) return launch_act<HYC_ACT_SILU>(g, stored, vals, scales, M, H, d, dx, stream, "hyc_act_bwd(silu)");
  if (act == HYC_ACT_GELU_TANH) return launch_act<HYC_ACT_GELU_TANH>(g, stored, vals, scales, M, H, d, dx, stream, "hyc_act_bwd(gelu)");
  return fail(HYC_EINVAL, "hyc_act_bwd: act=%d", act);
}

int hyc_hadamard_bwd(const void* g, const void* stored1, const void* vals1, const void* scales1, const hyc_desc* d1,
                     const void* stored2, const void* vals2, const void* scales2, const hyc_desc* d2, int64_t M,
                     int64_t H, void* dx1, void* dx2, void* stream) {
  // one pass when both operands use the channel scheme with the same code width and the row fits a workgroup
  if (d1 && d2 && d1->mode == HYC_MODE_CHANNEL && d2->mode == HYC_MODE_CHANNEL && d1->bits == d2->bits && d1->bits != 1 &&
      M > 0) {
    RowGeom geo;
    int rc = row_geom(H, d1->bits, &geo);
    if (rc) return rc;
    if (geo.iters == 1) {
      ChanArgs c1 = {}, c2 = {};
      int lpg = 16;
      if ((rc = make_chan_args(d1, geo, &c1, &lpg)) || (rc = make_chan_args(d2, geo, &c2, &lpg))) return rc;
      if (!g || !stored1 || !stored2 || !scales1 || !scales2 || !dx1 || !dx2 || (d1->k > 0 && !vals1) || (d2->k > 0 && !vals2))
        return fail(HYC_EFAULT, "hyc_hadamard_bwd: null buffer");
      if (!aligned16(g) || !aligned16(dx1) || !aligned16(dx2) || !aligned8(stored1) || !aligned8(stored2))
        return fail(HYC_EINVAL, "hyc_hadamard_bwd: g, dx must be 16-byte aligned, stored 8-byte");
      const int64_t cap = 256 * (geo.threads >= 512 ? 3 : 8);
      const int grid = row_loop_grid(M, cap, 4);
      hipStream_t st = begin_launch(stream);
#define HYC_HAD(B_, MT_)                                                                                           \
  hipLaunchKernelGGL((k_hadamard_bwd_fast<B_, MT_>), dim3(grid), dim3(geo.threads), 0, st,                         \
                     static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored1),                        \
                     static_cast<const uint16_t*>(vals1), static_cast<const uint16_t*>(scales1), c1,               \
                     static_cast<const uint8_t*>(stored2), static_cast<const uint16_t*>(vals2),                    \
                     static_cast<const uint16_t*>(scales2), c2, M, H, geo.cps, static_cast<uint16_t*>(dx1),        \
                     static_cast<uint16_t*>(dx2))
#define HYC_HAD_T(B_) do { if (geo.threads <= 256) HYC_HAD(B_, 256); else HYC_HAD(B_, 1024); } while (0)
      if (d1->bits == 2) HYC_HAD_T(2);
      else if (d1->bits == 4) HYC_HAD_T(4);
      else HYC_HAD_T(8);
#undef HYC_HAD_T
#undef HYC_HAD
      return check_launch("hyc_hadamard_bwd");
    }
  }
  int rc = launch_act<ACT_MUL>(g, stored2, vals2, scales2, M, H, d2, dx1, stream, "hyc_hadamard_bwd(dx1)");
  if (rc) return rc;
  return launch_act<ACT_MUL>(g, stored1, vals1, scales1, M, H, d1, dx2, stream, "hyc_hadamard_bwd(dx2)");
}

int hyc_gated_act_bwd(int32_t act, const void* g, const void* stored_a, const void* vals_a, const void* scales_a,
                      const hyc_desc* d_a, const void* stored_u, const void* vals_u, const void* scales_u,
                      const hyc_desc* d_u, const void* stored_g, const void* vals_g, const void* scales_g,
                      const hyc_desc* d_g, int64_t M, int64_t H, void* d_gate, void* d_up, void* stream) {
  if (act != HYC_ACT_SILU && act != HYC_ACT_GELU_TANH) return fail(HYC_EINVAL, "hyc_gated_act_bwd: act=%d", act);
  if (!d_a || !d_u || !d_g) return fail(HYC_EFAULT, "hyc_gated_act_bwd: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_gated_act_bwd: M=%lld", (long long)M);
  if (d_a->mode != HYC_MODE_CHANNEL || d_u->mode != HYC_MODE_CHANNEL || d_g->mode != HYC_MODE_CHANNEL)
    return fail(HYC_ENOTSUP, "hyc_gated_act_bwd: the three activations must be channel-compressed (use hyc_hadamard_bwd + hyc_act_bwd otherwise)");
  if (d_a->bits != d_u->bits || d_a->bits != d_g->bits || d_a->bits == 1)
    return fail(HYC_ENOTSUP, "hyc_gated_act_bwd: one code width (2, 4 or 8 bits) for the three activations");
  RowGeom geo;
  int rc = row_geom(H, d_a->bits, &geo);
  if (rc) return rc;
  if (geo.iters != 1) return fail(HYC_ENOTSUP, "hyc_gated_act_bwd: row too long (%d chunks per segment)", geo.cps);
  ChanArgs c_a = {}, c_u = {}, c_g = {};
  int lpg = 16;
  if ((rc = make_chan_args(d_a, geo, &c_a, &lpg)) || (rc = make_chan_args(d_u, geo, &c_u, &lpg)) ||
      (rc = make_chan_args(d_g, geo, &c_g, &lpg)))
    return rc;
  if (M == 0) return HYC_OK;
  if (!g || !stored_a || !stored_u || !stored_g || !scales_a || !scales_u || !scales_g || !d_gate || !d_up ||
      (d_a->k > 0 && !vals_a) || (d_u->k > 0 && !vals_u) || (d_g->k > 0 && !vals_g))
    return fail(HYC_EFAULT, "hyc_gated_act_bwd: null buffer");
  if (!aligned16(g) || !aligned16(d_gate) || !aligned16(d_up) || !aligned8(stored_a) || !aligned8(stored_u) || !aligned8(stored_g))
    return fail(HYC_EINVAL, "hyc_gated_act_bwd: g, d_gate, d_up must be 16-byte aligned, stored 8-byte");
  // rows of more than 768 chunks: two workgroups of the 768-thread variant per row where the row divides into whole
  // waves (the 1024-thread variant has 128 registers per thread and spills: 4096 x 14336, 113 us against 85)
  const int parts0 = geo.threads > 768 ? gated_row_parts(geo.cps, 768, lpg) : 1;
  const int parts = parts0 > 1 ? parts0 : 1;          // (no division into whole waves: the 1024-thread variant)
  const int cps_wg = geo.cps / parts, threads = parts > 1 ? ((cps_wg + 63) / 64) * 64 : geo.threads;
  // (workgroups of fewer than eight waves: fewer of them with more rows each, as for the activation backward - INT4,
  // 4096 x 4096, 2048 -> 768 workgroups: 30.7 -> 24.9 us; H = 5120, 2048 -> 512: 55.8 -> 44.0 us; INT2, 2048 -> 1024: 37.6 -> 33.7 us)
  // (from 32 768 rows on the tables are paid for either way and the resident grid is 2 % ahead: 394 against 403 us at 65 536)
  // Rows of eight waves or more: a CU holds one such workgroup at a time, so one per CU (and row part) with all its
  // rows beats three or four that each fill a table and start from an empty pipeline (4096 x 11008: 64.6 -> 60.1 us,
  // 2048 rows: 39.5 -> 32.8; the same at 16 384 rows; a grid that is not a multiple of the 256 CUs loses up to 15 %).
  const int64_t cap = threads * parts >= 512 ? 256 : M >= 32768 ? 2048 : threads <= 128 ? 1024 : threads <= 256 ? 768 : 512;
  const int gx = (int)(M < cap ? M : cap);
  const dim3 grid((unsigned)gx, (unsigned)(parts > 1 ? parts : 1));
  hipStream_t st = begin_launch(stream);
  const int use_lut = lut_pays(M, gx, threads, LUT_PAYS_OTHER);
#define HYC_GATED(B_, A_, MT_)                                                                                     \
  hipLaunchKernelGGL((k_gated_act_bwd_fast<B_, A_, MT_>), grid, dim3(threads), 0, st,                              \
                     static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored_a),                       \
                     static_cast<const uint16_t*>(vals_a), static_cast<const uint16_t*>(scales_a), c_a,            \
                     static_cast<const uint8_t*>(stored_u), static_cast<const uint16_t*>(vals_u),                  \
                     static_cast<const uint16_t*>(scales_u), c_u, static_cast<const uint8_t*>(stored_g),           \
                     static_cast<const uint16_t*>(vals_g), static_cast<const uint16_t*>(scales_g), c_g, M, H,      \
                     geo.cps, cps_wg, static_cast<uint16_t*>(d_gate), static_cast<uint16_t*>(d_up), use_lut)
#define HYC_GATED_T(B_, A_)                                                       \
  do {                                                                            \
    if (threads <= 256) HYC_GATED(B_, A_, 256);                                   \
    else if (threads <= 768) HYC_GATED(B_, A_, 768); /* H = 11008: 704 threads, 168 registers each */ \
    else HYC_GATED(B_, A_, 1024);                                                 \
  } while (0)
#define HYC_GATED_B(A_)                                                           \
  do {                                                                            \
    if (d_a->bits == 2) HYC_GATED_T(2, A_); else if (d_a->bits == 4) HYC_GATED_T(4, A_); else HYC_GATED_T(8, A_); \
  } while (0)
  if (act == HYC_ACT_SILU) HYC_GATED_B(HYC_ACT_SILU); else HYC_GATED_B(HYC_ACT_GELU_TANH);
#undef HYC_GATED_B
#undef HYC_GATED_T
#undef HYC_GATED
  return check_launch("hyc_gated_act_bwd");
}

int hyc_gated_act_fwd(int32_t act, const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int64_t M, int64_t H,
                      const hyc_desc* d_a, const hyc_desc* d_u, const hyc_desc* d_g, void* h, void* stored_a, void* vals_a,
                      void* scales_a, void* stored_u, void* vals_u, void* scales_u, void* stored_g, void* vals_g,
                      void* scales_g, void* stream) {
  if (act != HYC_ACT_SILU && act != HYC_ACT_GELU_TANH) return fail(HYC_EINVAL, "hyc_gated_act_fwd: act=%d", act);
  if (!d_a || !d_u || !d_g) return fail(HYC_EFAULT, "hyc_gated_act_fwd: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_gated_act_fwd: M=%lld", (long long)M);
  if (d_a->mode != HYC_MODE_CHANNEL || d_u->mode != HYC_MODE_CHANNEL || d_g->mode != HYC_MODE_CHANNEL)
    return fail(HYC_ENOTSUP, "hyc_gated_act_fwd: channel scheme only");
  if (d_a->bits != d_u->bits || d_a->bits != d_g->bits || d_a->group != d_u->group || d_a->group != d_g->group)
    return fail(HYC_ENOTSUP, "hyc_gated_act_fwd: one code width and one group size for the three activations");
  if (ld_gate < H || ld_up < H || ld_gate % 8 != 0 || ld_up % 8 != 0)
    return fail(HYC_EINVAL, "hyc_gated_act_fwd: row pitches %lld, %lld (at least H=%lld, multiples of 8)",
                (long long)ld_gate, (long long)ld_up, (long long)H);
  RowGeom geo;
  int rc = row_geom(H, d_a->bits, &geo);
  if (rc) return rc;
  ChanArgs c_a = {}, c_u = {}, c_g = {};
  int lpg = 16;
  if ((rc = make_chan_args(d_a, geo, &c_a, &lpg)) || (rc = make_chan_args(d_u, geo, &c_u, &lpg)) ||
      (rc = make_chan_args(d_g, geo, &c_g, &lpg)))
    return rc;
  // Three encoders side by side: the per-thread state grows with the segments a thread holds (four with 2-bit
  // codes), so the workgroup is capped at 768 threads (512 with 2-bit codes: 256 registers each); longer rows are
  // left to the separate calls.
  const int most = d_a->bits == 2 ? 512 : 768;
  const int parts = geo.iters == 1 ? (geo.threads > most ? gated_row_parts(geo.cps, most, lpg) : 1) : 0;
  if (parts == 0 || (d_a->bits != 2 && d_a->bits != 4 && d_a->bits != 8) || (lpg != 8 && lpg != 16))
    return fail(HYC_ENOTSUP, "hyc_gated_act_fwd: needs 2-, 4- or 8-bit codes, groups of 64 or 128 channels and rows of at "
                             "most 768 chunks per segment (512 with 2-bit codes), or up to 1024 that divide into 2 to 4 "
                             "such parts of whole scale groups (use the activation, hyc_compress and a product otherwise)");
  const int cps_wg = geo.cps / parts, threads = parts > 1 ? ((cps_wg + 63) / 64) * 64 : geo.threads;
  if (M == 0) return HYC_OK;
  if (!gate || !up || !h || !stored_a || !stored_u || !stored_g || !scales_a || !scales_u || !scales_g ||
      (d_a->k > 0 && !vals_a) || (d_u->k > 0 && !vals_u) || (d_g->k > 0 && !vals_g))
    return fail(HYC_EFAULT, "hyc_gated_act_fwd: null buffer");
  if (!aligned16(gate) || !aligned16(up) || !aligned16(h) || !aligned8(stored_a) || !aligned8(stored_u) || !aligned8(stored_g))
    return fail(HYC_EINVAL, "hyc_gated_act_fwd: gate, up, h must be 16-byte aligned, stored 8-byte");
  const GatedFwdSite sa = {c_a, static_cast<uint8_t*>(stored_a), static_cast<uint16_t*>(vals_a), static_cast<uint16_t*>(scales_a)};
  const GatedFwdSite su = {c_u, static_cast<uint8_t*>(stored_u), static_cast<uint16_t*>(vals_u), static_cast<uint16_t*>(scales_u)};
  const GatedFwdSite sg = {c_g, static_cast<uint8_t*>(stored_g), static_cast<uint16_t*>(vals_g), static_cast<uint16_t*>(scales_g)};
  const int64_t cap = 256 * (threads * parts >= 512 ? 3 : 8) / parts;
  // (rows of eight waves or more: one workgroup per CU and row part, as in the gated backward - 4096 x 11008:
  // 85.7 -> 79.1 us, 4096 x 14336: 124.9 -> 107.5, 2048 x 11008: 48.3 -> 40.0, 16 384 x 11008: 339 -> 321)
  const int gx = threads * parts >= 512 ? (int)(M < 256 ? M : 256) : (int)(M < cap ? M : cap);
  const dim3 grid((unsigned)gx, (unsigned)parts);
  hipStream_t st = begin_launch(stream);
  const int use_lut = lut_pays(M, gx, threads, LUT_PAYS_OTHER);
#define HYC_GFWD(B_, L_, A_, MT_)                                                                                  \
  hipLaunchKernelGGL((k_gated_act_fwd_fast<B_, L_, A_, MT_>), grid, dim3(threads), 0, st,                          \
                     static_cast<const uint16_t*>(gate), ld_gate, static_cast<const uint16_t*>(up), ld_up, M, H,   \
                     geo.cps, cps_wg, sa, su, sg, static_cast<uint16_t*>(h), use_lut)
#define HYC_GFWD_T(B_, L_, A_) /* H = 11008: 704 threads, up to 168 registers each */ \
  do { if (threads <= 256) HYC_GFWD(B_, L_, A_, 256); else HYC_GFWD(B_, L_, A_, 768); } while (0)
#define HYC_GFWD_L(B_, A_) do { if (lpg == 8) HYC_GFWD_T(B_, 8, A_); else HYC_GFWD_T(B_, 16, A_); } while (0)
#define HYC_GFWD_T2(L_, A_) do { if (threads <= 256) HYC_GFWD(2, L_, A_, 256); else HYC_GFWD(2, L_, A_, 512); } while (0)
#define HYC_GFWD_B(A_)                                                                                             \
  do {                                                                                                             \
    if (d_a->bits == 2) { if (lpg == 8) HYC_GFWD_T2(8, A_); else HYC_GFWD_T2(16, A_); }                            \
    else if (d_a->bits == 4) HYC_GFWD_L(4, A_); else HYC_GFWD_L(8, A_);                                           \
  } while (0)
  if (act == HYC_ACT_SILU) HYC_GFWD_B(HYC_ACT_SILU); else HYC_GFWD_B(HYC_ACT_GELU_TANH);
#undef HYC_GFWD_B
#undef HYC_GFWD_T2
#undef HYC_GFWD_L
#undef HYC_GFWD_T
#undef HYC_GFWD
  return check_launch("hyc_gated_act_fwd");
}

// shared host part of hyc_act_fwd_compress (x2 = NULL) and hyc_hadamard_fwd_compress
static int ew_fwd_impl(const char* who, int32_t act, const void* x1, int64_t ld1, const void* x2, int64_t ld2, int64_t M,
                       int64_t H, const hyc_desc* d1, const hyc_desc* d2, void* y, void* stored1, void* vals1, void* scales1,
                       void* stored2, void* vals2, void* scales2, void* stream) {
  const bool two = d2 != nullptr;
  if (!d1) return fail(HYC_EFAULT, "%s: null descriptor", who);
  if (M < 0) return fail(HYC_EINVAL, "%s: M=%lld", who, (long long)M);
  if (d1->mode != HYC_MODE_CHANNEL || (two && d2->mode != HYC_MODE_CHANNEL))
    return fail(HYC_ENOTSUP, "%s: channel scheme only", who);
  if (two && (d1->bits != d2->bits || d1->group != d2->group))
    return fail(HYC_ENOTSUP, "%s: one code width and one group size for both operands", who);
  if (ld1 < H || ld1 % 8 != 0 || (two && (ld2 < H || ld2 % 8 != 0)))
    return fail(HYC_EINVAL, "%s: row pitch (at least H=%lld, a multiple of 8)", who, (long long)H);
  RowGeom geo;
  int rc = row_geom(H, d1->bits, &geo);
  if (rc) return rc;
  ChanArgs c1 = {}, c2 = {};
  int lpg = 16;
  if ((rc = make_chan_args(d1, geo, &c1, &lpg)) || (two && (rc = make_chan_args(d2, geo, &c2, &lpg)))) return rc;
  // per-thread state grows with segments x operands: two operands of 2-bit codes take a workgroup of at most 512
  // threads (256 registers each)
  if (geo.iters != 1 || d1->bits == 1 || (two && d1->bits == 2 && geo.threads > 512) || (lpg != 8 && lpg != 16))
    return fail(HYC_ENOTSUP, "%s: needs 2-, 4- or 8-bit codes, groups of 64 or 128 channels and rows of at most 1024 "
                             "chunks per segment (512 for two operands of 2-bit codes; use the separate calls otherwise)", who);
  if (M == 0) return HYC_OK;
  if (!x1 || !y || !stored1 || !scales1 || (d1->k > 0 && !vals1) ||
      (two && (!x2 || !stored2 || !scales2 || (d2->k > 0 && !vals2))))
    return fail(HYC_EFAULT, "%s: null buffer", who);
  if (!aligned16(x1) || !aligned16(y) || !aligned8(stored1) || (two && (!aligned16(x2) || !aligned8(stored2))))
    return fail(HYC_EINVAL, "%s: inputs and y must be 16-byte aligned, stored 8-byte", who);
  const GatedFwdSite s1 = {c1, static_cast<uint8_t*>(stored1), static_cast<uint16_t*>(vals1), static_cast<uint16_t*>(scales1)};
  const GatedFwdSite s2 = {c2, static_cast<uint8_t*>(stored2), static_cast<uint16_t*>(vals2), static_cast<uint16_t*>(scales2)};
  const int64_t cap = 256 * (geo.threads >= 512 ? 3 : 8);
  int grid = row_loop_grid(M, cap, two ? 2 : 4);
  // (the erf form of GELU is the most expensive table to fill: wide rows take two workgroups per CU - 4096 x 11008:
  // 43.3 -> 39.4 us, 2048 rows: 25.8 -> 23.8, 16 384 rows: 176 -> 167; SiLU and the product keep the short loops)
  if (!two && act == HYC_ACT_GELU_TANH && geo.threads >= 512 && grid > 512) grid = 512;
  hipStream_t st = begin_launch(stream);
  const int use_lut = !two && lut_pays(M, grid, geo.threads, LUT_PAYS_OTHER);
#define HYC_EW(B_, L_, A_, N_, MT_)                                                                                \
  hipLaunchKernelGGL((k_ew_fwd_fast<B_, L_, A_, N_, MT_>), dim3(grid), dim3(geo.threads), 0, st,                   \
                     static_cast<const uint16_t*>(x1), ld1, static_cast<const uint16_t*>(x2), ld2, M, H, geo.cps,  \
                     s1, s2, static_cast<uint16_t*>(y), use_lut)
#define HYC_EW_T(B_, L_, A_, N_) do { if (geo.threads <= 256) HYC_EW(B_, L_, A_, N_, 256); else HYC_EW(B_, L_, A_, N_, 1024); } while (0)
#define HYC_EW_L(B_, A_, N_) do { if (lpg == 8) HYC_EW_T(B_, 8, A_, N_); else HYC_EW_T(B_, 16, A_, N_); } while (0)
  if (two && d1->bits == 2) {
    if (geo.threads <= 256) { if (lpg == 8) HYC_EW(2, 8, ACT_MUL, 2, 256); else HYC_EW(2, 16, ACT_MUL, 2, 256); }
    else { if (lpg == 8) HYC_EW(2, 8, ACT_MUL, 2, 512); else HYC_EW(2, 16, ACT_MUL, 2, 512); }
  } else if (two) {
    if (d1->bits == 4) HYC_EW_L(4, ACT_MUL, 2); else HYC_EW_L(8, ACT_MUL, 2);
  } else if (act == HYC_ACT_SILU) {
    if (d1->bits == 2) HYC_EW_L(2, HYC_ACT_SILU, 1); else if (d1->bits == 4) HYC_EW_L(4, HYC_ACT_SILU, 1); else HYC_EW_L(8, HYC_ACT_SILU, 1);
  } else {
    if (d1->bits == 2) HYC_EW_L(2, HYC_ACT_GELU_TANH, 1); else if (d1->bits == 4) HYC_EW_L(4, HYC_ACT_GELU_TANH, 1); else HYC_EW_L(8, HYC_ACT_GELU_TANH, 1);
  }
#undef HYC_EW_L
#undef HYC_EW_T
#undef HYC_EW
  return check_launch(who);
}

int hyc_act_fwd_compress(int32_t act, const void* x, int64_t ldx, int64_t M, int64_t H, const hyc_desc* d, void* y,
                         void* stored, void* vals, void* scales, void* stream) {
  if (act != HYC_ACT_SILU && act != HYC_ACT_GELU_TANH) return fail(HYC_EINVAL, "hyc_act_fwd_compress: act=%d", act);
  return ew_fwd_impl("hyc_act_fwd_compress", act, x, ldx, nullptr, 0, M, H, d, nullptr, y, stored, vals, scales, nullptr,
                     nullptr, nullptr, stream);
}

int hyc_hadamard_fwd_compress(const void* x1, int64_t ld1, const void* x2, int64_t ld2, int64_t M, int64_t H,
                              const hyc_desc* d1, const hyc_desc* d2, void* y, void* stored1, void* vals1, void* scales1,
                              void* stored2, void* vals2, void* scales2, void* stream) {
  if (!d2) return fail(HYC_EFAULT, "hyc_hadamard_fwd_compress: null descriptor");
  return ew_fwd_impl("hyc_hadamard_fwd_compress", 0, x1, ld1, x2, ld2, M, H, d1, d2, y, stored1, vals1, scales1, stored2,
                     vals2, scales2, stream);
}

}  // extern "C"
