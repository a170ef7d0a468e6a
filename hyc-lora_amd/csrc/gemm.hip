// Weight gradient of EfficientMemoryLinear:  dW[n, h] = sum_m dY[m, n] * x_hat[m, h]
// (reference: grad_output.transpose(-2, -1) @ x, operators/efficient_linear.py:56-67), with x_hat dequantised
// from the packed activation on the way into LDS - the decompressed [M, H] matrix never exists in HBM.
//
// MFMA v_mfma_f32_32x32x16_bf16, fp32 accumulation.  The reduction runs over tokens, and both operands are
// token-major in memory (a row = one token), so the LDS tiles are kept token-major as loaded and the 8-token
// operand fragments are gathered with the gfx950 transposing LDS read (ds_read_b64_tr_b16): inside a group of
// 16 lanes, lane i receives element (i mod 4) of the 8 bytes addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4.
//
// Because of the segment packing, one packed tile [tokens, 8c bytes] feeds NSEG separate ranges of output
// columns; a workgroup owns all of them so the packed bytes are read once.
#include <algorithm>
#include <utility>

#include "abi_util.hpp"
#include "row_kernels.hpp"

namespace hyc {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

constexpr int GK = 32;     // tokens per LDS stage
constexpr int GH = 128;    // output columns (channels) per workgroup
constexpr int GPAD = 16;   // row padding of the LDS tiles, in elements

__device__ __forceinline__ bf16x4_t tr_read(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
      (bf16x4_t __attribute__((address_space(3)))*)(const_cast<uint16_t*>(p)));
}

// Operand fragment of the 32 operand rows starting at column `col0` of a token-major tile T[token][pitch],
// tokens kk .. kk+15: lane L gets the 8 tokens kk + 8*(L/32) .. +7 of operand row L mod 32.
__device__ __forceinline__ bf16x8_t frag32(const uint16_t* T, int pitch, int col0, int kk) {
  const int lane = threadIdx.x & 63;
  const int g = lane >> 4, s = lane & 15;
  const uint16_t* p = T + (kk + 8 * (g >> 1) + (s >> 2)) * pitch + col0 + 16 * (g & 1) + 4 * (s & 3);
  const bf16x4_t lo = tr_read(p);
  const bf16x4_t hi = tr_read(p + 4 * pitch);
  bf16x8_t r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// SRC 0 = channel-compressed activation, 2 = dense bf16 activation.  BN = output rows (features of dY) per workgroup.
// grid: x = n-tile (fastest, so workgroups sharing an activation tile are neighbours), y = h-tile, z = token split.
template <int BITS, int SRC, int BN>
__global__ void __launch_bounds__(256)
k_gradw(const uint16_t* __restrict__ dy, int64_t ldy, int64_t M, int64_t N_out, int64_t H,
        const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals, const uint16_t* __restrict__ scales,
        ChanArgs ca, int CPS, int64_t tokens_per_split, float alpha, float beta, void* __restrict__ out, int out_f32,
        float* __restrict__ partial) {
  constexpr int NSEG = (SRC == 0) ? Q<BITS>::NSEG : 1;
  constexpr int HS = GH / NSEG;               // columns of the tile that come from one segment
  constexpr int CPR = HS / 8;                 // packed 8-byte chunks per token row of the tile
  constexpr int TN = (BN == 128) ? 2 : 1;     // 32x32 MFMA tiles per wave along n
  constexpr int TH = (BN == 128) ? 2 : 1;     // ... and along h
  constexpr int AP = BN + GPAD, BP = GH + GPAD;
  __shared__ __align__(16) uint16_t As[GK * AP];
  __shared__ __align__(16) uint16_t Bs[GK * BP];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int64_t n0 = (int64_t)blockIdx.x * BN;
  const int64_t SEG = (SRC == 0) ? (int64_t)CPS * 8 : H;
  const int64_t j0 = (int64_t)blockIdx.y * HS;          // first column of the tile inside each segment
  const int64_t m_begin = (int64_t)blockIdx.z * tokens_per_split;
  const int64_t m_end = m_begin + tokens_per_split < M ? m_begin + tokens_per_split : M;

  const int wn = (BN == 128) ? (wave >> 1) * 64 : 0;
  const int wh = (BN == 128) ? (wave & 1) * 64 : wave * 32;

  floatx16_t acc[TN][TH];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TH; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  constexpr int A_CHUNKS = GK * BN / 8;                   // 16-byte chunks of the dY tile
  constexpr int A_PER = (A_CHUNKS + 255) / 256;
  constexpr int B_ITEMS = GK * CPR;                       // packed chunks (SRC 0) or 16-byte chunks per segment (dense)
  constexpr int B_PER = (B_ITEMS + 255) / 256;

  for (int64_t m0 = m_begin; m0 < m_end; m0 += GK) {
    // ---- global -> registers -> LDS -------------------------------------------------------------------
    uint4 areg[A_PER];
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      const int idx = tid + u * 256;
      const int row = idx / (BN / 8), cc = idx % (BN / 8);
      const int64_t m = m0 + row, n = n0 + 8 * cc;
      areg[u] = (idx < A_CHUNKS && m < m_end && n < N_out) ? *reinterpret_cast<const uint4*>(dy + m * ldy + n)
                                                            : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();                                      // the previous stage has been consumed
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      const int idx = tid + u * 256;
      if (idx < A_CHUNKS) {
        const int row = idx / (BN / 8), cc = idx % (BN / 8);
        *reinterpret_cast<uint4*>(As + row * AP + 8 * cc) = areg[u];
      }
    }
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      const int idx = tid + u * 256;
      if (idx < B_ITEMS) {
        const int row = idx / CPR, cc = idx % CPR;
        const int64_t m = m0 + row;
        if (SRC == 0) {
          const int c = (int)(j0 / 8) + cc;               // chunk index inside a segment
          if (m < m_end) {
            const uint2 pk = *reinterpret_cast<const uint2*>(stored + m * SEG + 8 * c);
#pragma unroll
            for (int i = 0; i < NSEG; ++i) {
              *reinterpret_cast<uint4*>(Bs + row * BP + i * HS + 8 * cc) =
                  decode_chan_pk<BITS>(pk.x, pk.y, i, c, CPS, ca, vals + m * ca.k, scales + m * ca.groups_per_row);
            }
          } else {
#pragma unroll
            for (int i = 0; i < NSEG; ++i)
              *reinterpret_cast<uint4*>(Bs + row * BP + i * HS + 8 * cc) = make_uint4(0, 0, 0, 0);
          }
        } else {
          const uint16_t* xd = reinterpret_cast<const uint16_t*>(stored);
          *reinterpret_cast<uint4*>(Bs + row * BP + 8 * cc) =
              (m < m_end) ? *reinterpret_cast<const uint4*>(xd + m * H + j0 + 8 * cc) : make_uint4(0, 0, 0, 0);
        }
      }
    }
    __syncthreads();
    // ---- MFMA over the stage ------------------------------------------------------------------------------
#pragma unroll
    for (int kk = 0; kk < GK; kk += 16) {
      bf16x8_t af[TN], bfv[TH];
#pragma unroll
      for (int a = 0; a < TN; ++a) af[a] = frag32(As, AP, wn + 32 * a, kk);
#pragma unroll
      for (int b = 0; b < TH; ++b) bfv[b] = frag32(Bs, BP, wh + 32 * b, kk);
#pragma unroll
      for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TH; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bfv[b], acc[a][b], 0, 0, 0);
    }
  }

  // ---- epilogue: lane holds column (lane mod 32), rows 8*(v/4) + 4*(lane/32) + (v mod 4) of each 32x32 tile ----
  const bool direct = partial == nullptr;
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TH; ++b) {
      const int hl = wh + 32 * b + (lane & 31);              // column inside the tile
      const int64_t h = (int64_t)(hl / HS) * SEG + j0 + (hl % HS);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t n = n0 + wn + 32 * a + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (n < N_out) {
          const float val = acc[a][b][v];
          if (!direct) {
            partial[((int64_t)blockIdx.z * N_out + n) * H + h] = val;
          } else if (out_f32) {
            float* o = static_cast<float*>(out) + n * H + h;
            *o = (beta != 0.f) ? alpha * val + beta * *o : alpha * val;
          } else {
            uint16_t* o = static_cast<uint16_t*>(out) + n * H + h;
            *o = f_to_bf((beta != 0.f) ? alpha * val + beta * bf_to_f(*o) : alpha * val);
          }
        }
      }
    }
}


// ------------------------------------------------------------------------------------------------
// Few output rows (N_out <= 128: the LoRA-A shapes, dW [r, H], 32 features per workgroup): a streaming kernel without
// LDS tiles.
//
// v_mfma_f32_16x16x32_bf16: per lane 8 consecutive tokens of ONE row (A, a feature of dY) or ONE column (B, a
// channel of x_hat); lane L holds row/column L mod 16 and tokens 8*(L/16) .. +7 of the 32-token step.  A lane
// therefore owns one chunk (8 channels = the 8 code bytes of a packed word) and loads that chunk's word for its 8
// tokens; byte j of the 8 words is the operand fragment for channel 8c + j.  The 16 lanes of a quarter-wave own 16
// neighbouring chunks, so MFMA number j covers the 16 channels {8c + j}: a strided column set, which only permutes
// where results are stored.  The A operand is loaded the same way, one feature per lane.  A wave is self-contained
// (no barriers in the token loop, two steps of loads in flight); the four waves of a workgroup take every fourth
// step of the workgroup's token range and add their accumulators through LDS at the end.
//
// Outlier channels were quantised as zeros, so the main tiles contribute nothing there and do not store them;
// their columns dW[:, idx[q]] = dY^T vals[:, q] come from a second launch that feeds vals [M, k] to the same loop,
// 16 outlier channels per tile.
// ------------------------------------------------------------------------------------------------
constexpr int DK = 32;     // tokens per step = one MFMA k-step

typedef float floatx4_t __attribute__((ext_vector_type(4)));

// Buffer loads with a scalar offset on top of the lane's: the hardware checks the SUM of both offsets against the
// size of the resource, so a row selected through the scalar offset is dropped (reads zeros) when it lies past the end.
__device__ __forceinline__ uint4 load_b128(BufferRsrc r, uint32_t off, uint32_t scalar_off) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, (int)scalar_off, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_b64(BufferRsrc r, uint32_t off, uint32_t scalar_off) {
  const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, (int)scalar_off, 0);
  return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t load_b16(BufferRsrc r, uint32_t off, uint32_t scalar_off) {
  return (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(r, (int)off, (int)scalar_off, 0);
}

// Codes to floats, two per instruction.  A byte below 17 read as an FP8 number (E4M3, bias 7) is that integer times
// 2^-9: the exponent fields 0 and 1 share one step.  The scaled packed conversion multiplies by a power of two on
// its way (it takes the exponent of its scale operand), so with 2^9 the two bytes of one half of `w` come out as the
// floats of their integer values: exact, and half the instructions of one conversion per byte.  Serves every code
// width whose codes stay below 16.
template <bool HIGH_HALF>
__device__ __forceinline__ floatx2_t small_bytes_to_float(uint32_t w) {
  return __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(w, 512.f, HIGH_HALF);
}

struct DirectArgs {
  const uint16_t* dy; int64_t ldy, M, N_out, H;
  const uint8_t* stored; const uint16_t* vals; const uint16_t* scales;
  ChanArgs ca; int CPS, c_tiles; int64_t tokens_per_split;
  float alpha, beta; void* out; int out_f32; float* partial;
};

template <int SPT>
struct DirectRegs {          // what one lane loads for one step: a packed word and SPT group scales per token
  uint32_t blo[8], bhi[8], sc[SPT][8];
};

// MAINT: true = a tile of 16 chunks of SPT segments, decoded from the same packed words (which are then read once
//        per SPT segments); false = a tile of 16 outlier channels (bf16 values, nothing to decode)
// NT = 16-row tiles of dY features (N_out <= 16*NT)
// Every lane applies its own group scale: x_hat = bf16((code - OFF) * s), exactly what hyc_decompress writes.  (An
// earlier form folded the scale of 1- and 2-bit codes into dY, where code - OFF is exact, and fed the integer codes
// to the MFMAs as bf16 bit patterns; since the codes are converted two per instruction the plain form is as fast
// - 2-bit codes, 64-channel groups, 65 536 x 4096: 55.0 us folded, 41.8 us plain - and it went.)
// NW = waves per workgroup (4 or 8): the waves share the workgroup's token range step by step, so with eight a wave has
//      half as many steps to walk and the token range needs half as many splits across workgroups
template <int BITS, int NT, bool MAINT, int SPT, int NW>
__device__ __forceinline__ void gradw_direct_tile(const DirectArgs& A, float* red, int hy, int64_t n0) {
  constexpr int NTHR = 64 * NW;
  constexpr int LC = 16;                                                         // chunks per tile
  constexpr int NJ = 8;                                                          // MFMAs (16 channels each) per segment
  constexpr uint32_t CMASK = (BITS == 8) ? 0xFFu : Q<BITS>::CODE_MASK;
  constexpr uint32_t REP = CMASK * 0x01010101u;
  constexpr float OFFV = (BITS == 8) ? 128.f : (float)Q<BITS>::OFF;
  constexpr int NB = MAINT ? NJ * SPT : 1;                                       // 16-column MFMA tiles per wave
  constexpr int RP = 17;                                                         // padded pitch of the reduction buffer
  const ChanArgs& ca = A.ca;
  const int CPS = A.CPS, c_tiles = A.c_tiles;
  const int64_t ldy = A.ldy, N_out = A.N_out, H = A.H;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);                     // uniform: token bases stay scalar
  const int l16 = lane & 15, kq = lane >> 4;                                     // column / token quarter
  const int sgrp = MAINT ? hy / c_tiles : 0;                                     // group of SPT segments
  const int seg = sgrp * SPT;                                                    // its first segment
  const int c = MAINT ? (hy - sgrp * c_tiles) * LC + l16 : 0;                    // chunk inside the segment
  const int q = MAINT ? 0 : hy * 16 + l16;                                       // outlier number
  const int shs = (BITS == 8 || SPT == Q<BITS>::NSEG) ? 0 : seg * BITS;   // a tile of all segments starts at bit 0
  const int64_t m_begin = (int64_t)blockIdx.z * A.tokens_per_split;
  const int64_t m_end = m_begin + A.tokens_per_split < A.M ? m_begin + A.tokens_per_split : A.M;

  // Addresses = scalar base of (step, token e) + a 32-bit per-lane byte offset that never changes.
  const int64_t tok_b = MAINT ? (int64_t)CPS * 8 : (int64_t)ca.k * 2;            // bytes per token of the B source
  const int64_t sc_b = (int64_t)ca.groups_per_row * 2;
  const int64_t dy_b = ldy * 2;
  const char* bsrc = MAINT ? reinterpret_cast<const char*>(A.stored) : reinterpret_cast<const char*>(A.vals);
  const char* ssrc = reinterpret_cast<const char*>(A.scales);
  const char* asrc = reinterpret_cast<const char*>(A.dy);
  const int cc = c < CPS ? c : CPS - 1, qc = q < ca.k ? q : ca.k - 1;           // clamped: see fetch()
  const uint32_t lane_b = MAINT ? 8u * (uint32_t)cc : 2u * (uint32_t)qc;
  uint32_t lane_s[SPT];
#pragma unroll
  for (int g = 0; g < SPT; ++g) lane_s[g] = 2u * (uint32_t)(((seg + g) * CPS + cc) >> ca.chunk_to_group_shift);
  uint32_t lane_a[NT], aoff[NT];                                                 // feature 16a + l16, clamped
#pragma unroll
  for (int a = 0; a < NT; ++a) {
    lane_a[a] = 2u * (uint32_t)(n0 + 16 * a + l16 < N_out ? n0 + 16 * a + l16 : N_out - 1);
    aoff[a] = (uint32_t)(8 * kq * dy_b) + lane_a[a];
  }
  const uint32_t boff = (uint32_t)(8 * kq * tok_b) + lane_b;
  uint32_t soff[SPT];
#pragma unroll
  for (int g = 0; g < SPT; ++g) soff[g] = (uint32_t)(8 * kq * sc_b) + lane_s[g];

  // Where this thread will write at the end; its plan word (outlier mask of the chunk) or outlier channel index is
  // requested now, so that the load is over long before the write-out needs it.
  constexpr int COLS = MAINT ? SPT * LC * 8 : 16;                                // channels of the tile
  static_assert(COLS <= 256, "one thread per channel of the tile");
  const int mode = A.partial != nullptr ? 0 : (A.out_f32 ? 1 : 2);
  const bool wo_vec = MAINT && mode == 0;                                        // 4 channels per thread (the workspace is 16-byte aligned)
  const int wo_col = wo_vec ? (tid % (COLS / 4)) * 4 : tid % COLS;   // (NTHR is a multiple of COLS / 4 and of COLS)
  const int wo_tb = MAINT ? (wo_col & 7) : 0, wo_tcl = MAINT ? ((wo_col >> 3) % LC) : 0, wo_tg = MAINT ? wo_col / (8 * LC) : 0;
  bool wo_in;
  uint32_t wo_pword = 0;
  int64_t wo_h;
  if (MAINT) {
    const int tc = (hy - sgrp * c_tiles) * LC + wo_tcl;                          // chunk of this thread's channel(s)
    wo_in = tc < CPS;
    if (wo_in) wo_pword = ca.plan[(seg + wo_tg) * CPS + tc];
    wo_h = (int64_t)(seg + wo_tg) * CPS * 8 + 8 * tc + wo_tb;                    // a segment spans CPS*8 channels
  } else {
    wo_in = hy * 16 + wo_col < ca.k;
    wo_h = wo_in ? ca.idx[hy * 16 + wo_col] : 0;
  }

  floatx4_t acc[NT][NB];
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  // Every load is unconditional.  Lanes past the last chunk / outlier / feature read their neighbour's data (the
  // results are dropped at the write-out).  The buffer resources of a step span exactly its valid tokens, token e of
  // a lane's eight sits in the scalar offset (the hardware checks the sum of both offsets against the size), so
  // tokens past the end of the range read zeros: a zero dY operand, a zero scale.
  auto fetch = [&](int64_t m0, DirectRegs<SPT>& Rg, uint32_t (&ar)[NT][8]) __attribute__((always_inline)) {
    const uint32_t left = (uint32_t)(m_end - m0 < DK ? m_end - m0 : DK);        // valid tokens of the step
    const BufferRsrc rs_a = make_rsrc(asrc + m0 * dy_b, left * (uint32_t)dy_b);
    const BufferRsrc rs_b = make_rsrc(bsrc + m0 * tok_b, left * (uint32_t)tok_b);
    const BufferRsrc rs_s = make_rsrc(ssrc + m0 * sc_b, left * (uint32_t)sc_b);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (MAINT) {
        const uint2 w = load_b64(rs_b, boff, (uint32_t)e * (uint32_t)tok_b);
        Rg.blo[e] = w.x; Rg.bhi[e] = w.y;
#pragma unroll
        for (int g = 0; g < SPT; ++g) Rg.sc[g][e] = load_b16(rs_s, soff[g], (uint32_t)e * (uint32_t)sc_b);
      } else {
        Rg.blo[e] = load_b16(rs_b, boff, (uint32_t)e * (uint32_t)tok_b);
      }
#pragma unroll
      for (int a = 0; a < NT; ++a) ar[a][e] = load_b16(rs_a, aoff[a], (uint32_t)e * (uint32_t)dy_b);
    }
  };
  auto step = [&](DirectRegs<SPT>& Rg, uint32_t (&ar)[NT][8]) __attribute__((always_inline)) {
    bf16x8_t af[NT];
#pragma unroll
    for (int a = 0; a < NT; ++a)
      af[a] = __builtin_bit_cast(bf16x8_t, (u32x4_t){ar[a][0] | (ar[a][1] << 16), ar[a][2] | (ar[a][3] << 16),
                                                     ar[a][4] | (ar[a][5] << 16), ar[a][6] | (ar[a][7] << 16)});
    if (MAINT) {
#pragma unroll
      for (int g = 0; g < SPT; ++g) {                  // one segment at a time: decode its 8 fragments, then their MFMAs
        bf16x8_t bfrag[8];
        float s[8], ns[8];
        uint32_t clo[8], chi[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          s[e] = bf_to_f((uint16_t)Rg.sc[g][e]); ns[e] = -OFFV * s[e];
          // segment seg + g's code of every byte, as a byte
          clo[e] = (BITS == 8) ? Rg.blo[e] ^ 0x80808080u : (Rg.blo[e] >> (shs + g * BITS)) & REP;
          chi[e] = (BITS == 8) ? Rg.bhi[e] ^ 0x80808080u : (Rg.bhi[e] >> (shs + g * BITS)) & REP;
          // opaque from here on: each code then costs one byte-to-float conversion; left visible, the compiler folds
          // this mask into one bit-field extract per code ahead of the conversion
          asm volatile("" : "+v"(clo[e]), "+v"(chi[e]));
        }
        if (BITS <= 4) {
          // two neighbouring bytes of a token's word per conversion; a fragment register wants two tokens of one byte
#pragma unroll
          for (int j = 0; j < 8; j += 2) {
            uint32_t w0[4], w1[4];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              floatx2_t p[2];
#pragma unroll
              for (int d = 0; d < 2; ++d) {
                const uint32_t w = (j < 4) ? clo[e + d] : chi[e + d];
                p[d] = (j & 2) ? small_bytes_to_float<true>(w) : small_bytes_to_float<false>(w);
              }
              w0[e >> 1] = pack_bf16(__builtin_fmaf(p[0].x, s[e], ns[e]), __builtin_fmaf(p[1].x, s[e + 1], ns[e + 1]));
              w1[e >> 1] = pack_bf16(__builtin_fmaf(p[0].y, s[e], ns[e]), __builtin_fmaf(p[1].y, s[e + 1], ns[e + 1]));
            }
            bfrag[j] = __builtin_bit_cast(bf16x8_t, (u32x4_t){w0[0], w0[1], w0[2], w0[3]});
            bfrag[j + 1] = __builtin_bit_cast(bf16x8_t, (u32x4_t){w1[0], w1[1], w1[2], w1[3]});
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            uint32_t wj[4];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              float f[2];
#pragma unroll
              for (int d = 0; d < 2; ++d) {
                const uint32_t w = (j < 4) ? clo[e + d] : chi[e + d];
                f[d] = __builtin_fmaf((float)((w >> (8 * (j & 3))) & 0xFFu), s[e + d], ns[e + d]);
              }
              wj[e >> 1] = pack_bf16(f[0], f[1]);
            }
            bfrag[j] = __builtin_bit_cast(bf16x8_t, (u32x4_t){wj[0], wj[1], wj[2], wj[3]});
          }
        }
#pragma unroll
        for (int a = 0; a < NT; ++a)
#pragma unroll
          for (int j = 0; j < 8; ++j)
            acc[a][8 * g + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[a], bfrag[j], acc[a][8 * g + j], 0, 0, 0);
        if (g + 1 < SPT) __builtin_amdgcn_sched_barrier(0);   // keep the segments apart: decoding both first spills
      }
    } else {
      const bf16x8_t bfrag = __builtin_bit_cast(bf16x8_t, (u32x4_t){Rg.blo[0] | (Rg.blo[1] << 16), Rg.blo[2] | (Rg.blo[3] << 16),
                                                                   Rg.blo[4] | (Rg.blo[5] << 16), Rg.blo[6] | (Rg.blo[7] << 16)});
#pragma unroll
      for (int a = 0; a < NT; ++a) acc[a][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[a], bfrag, acc[a][0], 0, 0, 0);
    }
  };

  // wave w takes steps w, w+NW, ... of the workgroup's token range; two steps of loads are in flight
  constexpr int64_t WS = NW * DK;
  DirectRegs<SPT> R0, R1;
  uint32_t a0[NT][8], a1[NT][8];
  int64_t m0 = m_begin + (int64_t)wave * DK;
  if (m0 < m_end) fetch(m0, R0, a0);
  if (m0 + WS < m_end) fetch(m0 + WS, R1, a1);
  for (; m0 < m_end; m0 += 2 * WS) {
    step(R0, a0);
    if (m0 + 2 * WS < m_end) fetch(m0 + 2 * WS, R0, a0);
    if (m0 + WS < m_end) {
      step(R1, a1);
      if (m0 + 3 * WS < m_end) fetch(m0 + 3 * WS, R1, a1);
    }
  }
  // ---- the waves add up in LDS: the first half of them write their accumulators to a buffer each, the second half
  // add theirs on top (wave w onto wave w - NW/2), and the write-out adds the NW/2 buffers; layout of a buffer
  // [row n][tile b][lane] with a padded pitch ----
  // lane holds column (lane mod 16) and rows 4*(lane/16) + v of each 16x16 tile
  constexpr int NBUF = NW / 2;
  constexpr int HALF = 16 * NT * NB * RP;                                        // floats of one buffer
  float* mine = red + (wave % NBUF) * HALF;
  if (wave < NBUF) {
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) mine[((16 * a + 4 * kq + v) * NB + b) * RP + l16] = acc[a][b][v];
  }
  __syncthreads();
  if (wave >= NBUF) {
    // all reads first, then the adds and writes: written as read-add-write per element the compiler keeps them in
    // program order (it cannot see that the addresses differ) and every element waits out the LDS latency
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[a][b][v] += mine[((16 * a + 4 * kq + v) * NB + b) * RP + l16];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) mine[((16 * a + 4 * kq + v) * NB + b) * RP + l16] = acc[a][b][v];
  }
  __syncthreads();
  // sum of the buffers at one place, in buffer order
  auto reduced = [&](int at) __attribute__((always_inline)) {
    float v = red[at];
#pragma unroll
    for (int u = 1; u < NBUF; ++u) v += red[u * HALF + at];
    return v;
  };
  // ---- write-out by all threads, neighbouring threads = neighbouring channels ----
  const float alpha = A.alpha, beta = A.beta;
  if (!wo_in) return;
  // channel = (segment tg of the tile, chunk tcl of the tile, byte tb of the packed word): MFMA tile 8*tg + tb, lane tcl
  if (wo_vec) {                                        // partial sums of a main tile: 16-byte stores, 4 channels per thread
    constexpr int NSTEP4 = NTHR / (COLS / 4);
    int ro[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ro[i] = (wo_tg * NJ + wo_tb + i) * RP + wo_tcl;
    const uint32_t m4 = (wo_pword >> wo_tb) & 0xFu;    // outlier channels belong to the outlier tiles
    for (int nl = tid / (COLS / 4); nl < 16 * NT && n0 + nl < N_out; nl += NSTEP4) {
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = reduced(nl * NB * RP + ro[i]);
      float* o = A.partial + ((int64_t)blockIdx.z * N_out + n0 + nl) * H + wo_h;
      if (m4 == 0) {
        *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (!((m4 >> i) & 1u)) o[i] = v[i];
      }
    }
    return;
  }
  if (MAINT && ((wo_pword >> wo_tb) & 1u)) return;
  const int rb = MAINT ? wo_tg * NJ + wo_tb : 0, rl = MAINT ? wo_tcl : tid % COLS;
  for (int nl = tid / COLS; nl < 16 * NT && n0 + nl < N_out; nl += NTHR / COLS) {
    const float val = reduced((nl * NB + rb) * RP + rl);
    const int64_t n = n0 + nl;
    if (mode == 0) {
      A.partial[((int64_t)blockIdx.z * N_out + n) * H + wo_h] = val;
    } else if (mode == 1) {
      float* o = static_cast<float*>(A.out) + n * H + wo_h;
      *o = (beta != 0.f) ? alpha * val + beta * *o : alpha * val;
    } else {
      uint16_t* o = static_cast<uint16_t*>(A.out) + n * H + wo_h;
      *o = f_to_bf((beta != 0.f) ? alpha * val + beta * bf_to_f(*o) : alpha * val);
    }
  }
}

// one launch: blockIdx.y < (NSEG / SPT) * c_tiles are the tiles of quantised channels, the rest the outlier tiles
// (two waves per SIMD at least: with 256 registers or fewer the accumulators stay in ordinary vector registers)
template <int BITS, int NT, int SPT, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) k_gradw_direct(DirectArgs A) {
  static_assert(Q<BITS>::NSEG % SPT == 0, "segments per tile must divide the segments of a packed word");
  constexpr int NB = 8 * SPT;
  __shared__ float red[(NW / 2) * 16 * NT * NB * 17];
  const int main_tiles = (Q<BITS>::NSEG / SPT) * A.c_tiles;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * NT);                            // first feature of the workgroup
  if ((int)blockIdx.y < main_tiles) gradw_direct_tile<BITS, NT, true, SPT, NW>(A, red, (int)blockIdx.y, n0);
  else gradw_direct_tile<BITS, NT, false, 1, NW>(A, red, (int)blockIdx.y - main_tiles, n0);
}

// How a shape is laid on the kernel: SPT segments of a packed word per tile (two with one feature tile, so that every
// word is loaded once; the accumulators of two feature tiles leave room for one), and how many workgroups of the
// variant a CU holds at once (three where it needs at most 168 registers per lane, else two).
struct DirectPlan { int spt, per_cu; };
static DirectPlan direct_plan(int bits, int64_t N_out) {
  DirectPlan p;
  const int nseg = 8 / bits, nt = N_out <= 16 ? 1 : 2;
  p.spt = nt == 1 && nseg >= 2 ? 2 : 1;
  p.per_cu = (nt == 1 && p.spt == 1) ? 3 : 2;
  return p;
}

// The streaming kernel serves N_out <= DIRECT_MAX_N.  The token splits keep the whole grid resident at once
// (256 CUs x the workgroups a CU holds): the kernel is bound by its decode work, so a grid a little over that
// leaves most of the chip idle during a second round (65 536 x 4096 INT4, two per CU: 560 workgroups 88 us, 490
// workgroups 65 us).
// More than 32 features run as blockIdx.x tiles of 32 that decode the packed words again: up to four such tiles
// that still beats staging the tile in LDS for a product this thin.
constexpr int64_t DIRECT_MAX_N = 128;
static int64_t direct_x_tiles(int64_t N_out) { return N_out <= 32 ? 1 : (N_out + 31) / 32; }
// Token splits for workgroups of nw waves: as many as keep the whole grid resident at once (two workgroups of four
// waves per CU, or one of eight), and no more than leave every wave two steps of 32 tokens (four for four waves from
// 4096 tokens on: a split more is a partial result more for the second launch to add - 4096 x 16 x 4096: 16 splits
// 12.1 us, 8 splits 11.3; 2048 tokens: 8 splits 9.3 us, 6 splits 11.6).
static int direct_splits(int64_t M, int64_t yx_tiles, int nw, int per_cu4) {
  const int per_cu = nw == 8 ? 1 : per_cu4;               // (per_cu4: workgroups of four waves a CU holds, see direct_plan)
  int64_t s = (int64_t)256 * per_cu / (yx_tiles > 0 ? yx_tiles : 1);
  const int64_t per_wave = nw == 8 ? 2 : M >= 4096 ? 4 : M >= 3072 ? 3 : 2;
  const int64_t max_by_tokens = (M + nw * per_wave * DK - 1) / (nw * per_wave * DK);
  if (s > max_by_tokens) s = max_by_tokens;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return (int)s;
}
// Waves per workgroup.  Eight waves walk a token range in half the steps and need half the splits (fewer partial
// results to add): better wherever the kernel is short (4096 x 16 x 4096 4-bit: 10.6 us against 11.3, r = 64: 14.7
// against 16.3, 11008 channels: 14.4 against 15.6).  With many steps per wave what counts is how much of the chip the
// grid fills, and the two forms fill it in different grains (65 536 x 64 x 4096: 210 workgroups of eight waves, 109 us,
// against 490 of four, 95 us); below 4096 tokens the larger reduction through LDS costs more than the steps saved
// (2048 tokens: 11.2 against 9.3 us).
static int direct_waves(int64_t M, int64_t yx_tiles, int per_cu4) {
  if (M < 4096) return 4;
  const int s8 = direct_splits(M, yx_tiles, 8, per_cu4), s4 = direct_splits(M, yx_tiles, 4, per_cu4);
  const int64_t steps8 = (M + (int64_t)s8 * 8 * DK - 1) / ((int64_t)s8 * 8 * DK);
  if (steps8 <= 8) return 8;
  return yx_tiles * s8 * 8 >= yx_tiles * s4 * 4 ? 8 : 4;      // waves in flight
}
static int64_t direct_y_tiles(int64_t H, int bits, int k, int64_t N_out) {
  const DirectPlan p = direct_plan(bits, N_out);
  const int64_t cps = (H * bits + 63) / 64;
  return (8 / bits / p.spt) * ((cps + 15) / 16) + (k + 15) / 16;
}
// the most splits any code width can ask for (the workspace query does not know it)
static int direct_splits_max(int64_t M, int64_t N_out, int64_t H) {
  int best = 1;
  for (int bits = 1; bits <= 8; bits *= 2) {
    const int sp = direct_splits(M, direct_y_tiles(H, bits, 0, N_out) * direct_x_tiles(N_out), 4, direct_plan(bits, N_out).per_cu);   // (four waves: the form with more splits)
    if (sp > best) best = sp;
  }
  return best;
}

// ------------------------------------------------------------------------------------------------
// Large output (N_out > 32), first form: workgroup tile 128 (n) x 256 (h), four waves of 64 x 128, two LDS stages.
// While the MFMAs of stage s run, the global loads of stage s+1 are in flight; they are written into the other LDS
// buffer after the MFMAs have been issued, and one barrier per stage separates the two.  128 accumulator registers
// per lane and two waves per SIMD.  For a dense activation whose tile grid is too small for the 256-feature form
// below.
// ------------------------------------------------------------------------------------------------
constexpr int WK = 32;      // tokens per stage
constexpr int WN = 128;     // dY features per workgroup of this form (the second form takes 2 * WN)
constexpr int WH = 256;     // channels per workgroup
constexpr int WPAD = 32;    // row padding of the wide kernel's LDS tiles, in elements

template <int NSEG, int A_PER, int B_PER>
struct WideRegs {            // one stage of global data per thread
  uint4 a[A_PER];            // dY chunks
  uint4 b[B_PER];            // channel scheme: .x/.y = packed word; dense: 8 bf16
  uint32_t s[B_PER][NSEG];   // channel scheme: the group scale of each segment's chunk
  uint32_t o0[B_PER][NSEG], o1[B_PER][NSEG];   // ... and the first two outlier values of the chunk
};

// dense activation only (x = bf16 [M, H]); grid: x = n-tile, y = h-tile, z = token split
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
k_gradw_wide(const uint16_t* __restrict__ dy, int64_t ldy, int64_t M, int64_t N_out, int64_t H,
             const uint16_t* __restrict__ x, int64_t tokens_per_split, float alpha, float beta,
             void* __restrict__ out, int out_f32, float* __restrict__ partial) {
  constexpr int CPR = WH / 8;                 // 16-byte chunks per token row of the x tile
  constexpr int THREADS = 2 * WN;             // four waves: 2 along n x 2 along h, 64 x 128 each
  constexpr int AP = WN + WPAD, BP = WH + WPAD;
  __shared__ __align__(16) uint16_t As[2][WK * AP];
  __shared__ __align__(16) uint16_t Bs[2][WK * BP];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t n0 = (int64_t)blockIdx.x * WN;
  const int64_t j0 = (int64_t)blockIdx.y * WH;
  const int64_t m_begin = (int64_t)blockIdx.z * tokens_per_split;
  const int64_t m_end = m_begin + tokens_per_split < M ? m_begin + tokens_per_split : M;
  const int wn = (wave >> 1) * 64, wh = (wave & 1) * 128;

  floatx16_t acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  constexpr int A_PER = WK * WN / 8 / THREADS;            // 16-byte chunks of the dY stage per thread (2)
  constexpr int B_PER = WK * CPR / THREADS;               // ... and of the x stage (4)
  typedef WideRegs<1, A_PER, B_PER> Regs;
  // Every operand of the token loop is read through a buffer resource that spans exactly this workgroup's token
  // range: the hardware drops what lies beyond it (rows past m_end, features past N_out) and returns zeros, so
  // nothing is clamped, predicated or branched on, and the address of a load is a per-thread constant.
  const uint32_t b_pitch = 2u * (uint32_t)H;
  uint32_t va[A_PER], vb[B_PER];
#pragma unroll
  for (int u = 0; u < A_PER; ++u) {
    const int idx = tid + u * THREADS;
    const int row = idx / (WN / 8), cc = idx % (WN / 8);
    va[u] = n0 + 8 * cc < N_out ? 2u * ((uint32_t)row * (uint32_t)ldy + (uint32_t)n0 + 8u * cc) : NOWHERE;
  }
#pragma unroll
  for (int u = 0; u < B_PER; ++u) {
    const int idx = tid + u * THREADS;
    vb[u] = (uint32_t)(idx / CPR) * b_pitch + 2u * ((uint32_t)j0 + 8u * (idx % CPR));
  }
  auto fetch = [&](Regs& R, int64_t m0) __attribute__((always_inline)) {
    // the resources of a stage start at its first token (scalar arithmetic), so the per-thread offsets never change
    const uint32_t left = (uint32_t)(m_end - m0);
    const BufferRsrc rs_a = make_rsrc(dy + m0 * ldy, left * 2u * (uint32_t)ldy);
    const BufferRsrc rs_b = make_rsrc(x + m0 * H, left * b_pitch);
#pragma unroll
    for (int u = 0; u < A_PER; ++u) R.a[u] = load_b128(rs_a, va[u]);
#pragma unroll
    for (int u = 0; u < B_PER; ++u) R.b[u] = load_b128(rs_b, vb[u]);
  };
  auto stash = [&](int buf, const Regs& R) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) {
      const int idx = tid + u * THREADS;
      *reinterpret_cast<uint4*>(&As[buf][(idx / (WN / 8)) * AP + 8 * (idx % (WN / 8))]) = R.a[u];
    }
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      const int idx = tid + u * THREADS;
      *reinterpret_cast<uint4*>(&Bs[buf][(idx / CPR) * BP + 8 * (idx % CPR)]) = R.b[u];
    }
  };
  // The 16 MFMAs of a stage run as 8 pairs (k sub-step t/4, column tile t%4; both row tiles of the wave).  Operand
  // fragments are fetched two pairs ahead of their use (a ring of four B fragments, the A fragments of the second
  // sub-step during the first), so the LDS latency sits under the MFMAs already issued.
  auto mfma_stage = [&](int buf) __attribute__((always_inline)) {
    bf16x8_t af[2][2], bq[4];
    af[0][0] = frag32(As[buf], AP, wn, 0);
    af[0][1] = frag32(As[buf], AP, wn + 32, 0);
    bq[0] = frag32(Bs[buf], BP, wh, 0);
    bq[1] = frag32(Bs[buf], BP, wh + 32, 0);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      __builtin_amdgcn_sched_barrier(0);
      if (t + 2 < 8) bq[(t + 2) & 3] = frag32(Bs[buf], BP, wh + 32 * ((t + 2) & 3), 16 * ((t + 2) >> 2));
      if (t == 1) {
        af[1][0] = frag32(As[buf], AP, wn, 16);
        af[1][1] = frag32(As[buf], AP, wn + 32, 16);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < 2; ++a)
        acc[a][t & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[t >> 2][a], bq[t & 3], acc[a][t & 3], 0, 0, 0);
    }
  };

  // Three stages in flight: stage s in LDS under the MFMAs, stage s+1 in registers on its way into the other LDS
  // buffer, stage s+2 on its way from memory.  One barrier per stage.
  if (m_begin < m_end) {
    Regs R0, R1;
    int64_t m0 = m_begin;
    fetch(R0, m0);
    stash(0, R0);
    if (m0 + WK < m_end) fetch(R0, m0 + WK);
    for (; m0 < m_end; m0 += 2 * WK) {
      if (m0 + 2 * WK < m_end) fetch(R1, m0 + 2 * WK);
      __syncthreads();                                    // buffer 0 is complete; buffer 1 is no longer read
      if (m0 + WK < m_end) stash(1, R0);
      mfma_stage(0);
      if (m0 + WK < m_end) {
        if (m0 + 3 * WK < m_end) fetch(R0, m0 + 3 * WK);
        __syncthreads();
        if (m0 + 2 * WK < m_end) stash(0, R1);
        mfma_stage(1);
      }
    }
  }

  // ---- epilogue: lane holds column (lane mod 32), rows 8*(v/4) + 4*(lane/32) + (v mod 4) of each 32x32 tile ----
  const bool direct = partial == nullptr;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int64_t h = j0 + wh + 32 * b + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t n = n0 + wn + 32 * a + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (n < N_out) {
          const float val = acc[a][b][v];
          if (!direct) {
            partial[((int64_t)blockIdx.z * N_out + n) * H + h] = val;
          } else if (out_f32) {
            float* o = static_cast<float*>(out) + n * H + h;
            *o = (beta != 0.f) ? alpha * val + beta * *o : alpha * val;
          } else {
            uint16_t* o = static_cast<uint16_t*>(out) + n * H + h;
            *o = f_to_bf((beta != 0.f) ? alpha * val + beta * bf_to_f(*o) : alpha * val);
          }
        }
      }
    }
}

// ------------------------------------------------------------------------------------------------
// Large output, second form: workgroup tile 256 (n) x 256 (h) on FOUR waves of 128 x 128, one per SIMD.  A wave's 256
// fp32 accumulators live in the accumulation registers (the compiler puts them there by itself at one wave per SIMD),
// which leaves the 256 ordinary registers to operand fragments and to the data of the next three stages.  Against the
// 64 x 128 wave tile of the first form this halves the operand bytes read from LDS per MFMA (8 fragments per 16
// MFMAs instead of 6 per 8).  With a single wave per SIMD nothing but the wave's own next instructions can fill the
// 32 cycles of an MFMA (eight issue slots: the MFMA and seven others; measured: up to six ordinary VALU instructions
// hide under one), so a stage of 32 tokens is laid out by hand as 32 slots, one MFMA each:
//   slots  0- 7  read the fragments of the stage's second 16 tokens
//   slots  0-15  decode stage s+1 (two elements per slot; its registers were requested two stages ago)
//   slots  8-15  request stage s+3 into the register set that held stage s
//   slots 16-23  write stage s+1 to the next LDS buffer, move the buffer resources on
//   slot  24     the stage's one barrier; slots 24-31 read the fragments of the first 16 tokens of stage s+1 and
//                prepare the decode of stage s+2 (code bytes, scales)
// ------------------------------------------------------------------------------------------------
template <int V> struct StageNo { static constexpr int value = V; };
// f(StageNo<0>), f(StageNo<1>), ... : a loop whose bodies are separate instantiations (no unroll threshold applies)
template <class F, int... T>
__device__ __forceinline__ void for_each_slot(F&& f, std::integer_sequence<int, T...>) { (f(StageNo<T>{}), ...); }

template <int BITS, int SRC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
k_gradw_big(const uint16_t* __restrict__ dy, int64_t ldy, int64_t M, int64_t N_out, int64_t H,
            const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals, const uint16_t* __restrict__ scales,
            ChanArgs ca, int CPS, int64_t tokens_per_split, float alpha, float beta,
            void* __restrict__ out, int out_f32, float* __restrict__ partial) {
  constexpr int NSEG = (SRC == 0) ? Q<BITS>::NSEG : 1;
  constexpr int TN = 256;                     // dY features per workgroup
  constexpr int HS = WH / NSEG;               // columns of the tile that come from one segment
  constexpr int CPR = HS / 8;                 // packed 8-byte chunks (channel scheme) / 16-byte chunks (dense) per token row and segment
  constexpr int THREADS = 256;
  constexpr int AP = TN + WPAD, BP = WH + WPAD;
  constexpr int NBUF = 3;
  __shared__ __align__(16) uint16_t lds[NBUF * WK * (AP + BP)];
#define HYC_AS(b_) (lds + (b_) * (WK * AP))
#define HYC_BS(b_) (lds + NBUF * (WK * AP) + (b_) * (WK * BP))

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Which tile: workgroups are dealt to the 8 XCDs in turn (workgroup L of a launch runs on XCD L mod 8) and every XCD
  // has an L2 of its own, so XCD q takes a contiguous run of tiles in an order that walks 4 feature tiles by all
  // channel tiles: its workgroups then share 4 dY panels and a short run of x_hat panels instead of 2 and all of them
  // (1-4 % on real operands: 4096 x 4096 x 11008 dense 328 -> 320 us, INT2 4096^3 138 -> 132 us).
  int tile_n = (int)blockIdx.x, tile_h = (int)blockIdx.y;
  {
    const int gx = (int)gridDim.x, gy = (int)gridDim.y, T = gx * gy;
    if (T % 8 == 0 && gx % 4 == 0) {
      const int L = tile_n + gx * tile_h;
      const int t = (L % 8) * (T / 8) + L / 8;
      const int band = t / (4 * gy), r = t - band * (4 * gy);
      tile_n = band * 4 + r % 4;
      tile_h = r / 4;
    }
  }
  const int64_t n0 = (int64_t)tile_n * TN;
  const int64_t SEG = (SRC == 0) ? (int64_t)CPS * 8 : H;
  const int64_t j0 = (int64_t)tile_h * HS;              // first column of the tile inside each segment
  const int64_t m_begin = (int64_t)blockIdx.z * tokens_per_split;
  const int64_t m_end = m_begin + tokens_per_split < M ? m_begin + tokens_per_split : M;
  const int wn = (wave >> 1) * 128, wh = (wave & 1) * 128;

  floatx16_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  constexpr int A_PER = WK * TN / 8 / THREADS;            // 16-byte chunks of the dY stage per thread (4)
  constexpr int B_ITEMS = WK * CPR;
  constexpr int B_PER = (B_ITEMS + THREADS - 1) / THREADS;
  static_assert(B_ITEMS % THREADS == 0 || B_ITEMS < THREADS, "items per stage");
  // Narrow codes give fewer packed words per stage than threads: PARTS threads then share a word, NST segments each.
  constexpr int PARTS = (SRC == 0 && B_ITEMS < THREADS) ? THREADS / B_ITEMS : 1;
  constexpr int NST = NSEG / PARTS;                       // segments a thread decodes
  static_assert(NSEG % PARTS == 0 && (PARTS == 1 || PARTS * B_ITEMS == THREADS), "threads per packed word");
  constexpr int NCH = B_PER * NST;                        // 16-byte chunks of the x stage per thread
  static_assert(A_PER == 4 && NCH == 4, "the slot plan below is written for four chunks of either operand");
  const int seg0 = (PARTS > 1 ? tid / B_ITEMS : 0) * NST; // first of them
  const int item0 = PARTS > 1 ? tid % B_ITEMS : tid;      // the thread's first item
  typedef WideRegs<NST, A_PER, B_PER> Regs;
  ChunkOutliers<NST> co;
  {
    uint32_t pw[NST];
#pragma unroll
    for (int i = 0; i < NST; ++i)
      pw[i] = (SRC == 0) ? ca.plan[(seg0 + i) * CPS + (int)(j0 / 8) + item0 % CPR] : 0u;
    co.init(pw);
  }

  // Every operand of the token loop is read through a buffer resource that starts at the stage's first token and
  // ends with the workgroup's token range: nothing is clamped, predicated or branched on, a stage past the end
  // reads zeros, and the addresses are per-thread constants.
  const uint32_t gpr = (uint32_t)ca.groups_per_row, kk2 = 2u * (uint32_t)ca.k;
  const uint32_t a_pitch = 2u * (uint32_t)ldy;
  const uint32_t b_pitch = (SRC == 0) ? (uint32_t)SEG : 2u * (uint32_t)H;          // bytes per token of the x operand
  uint32_t va[A_PER], vb[B_PER], vs[B_PER][NST], vo0[B_PER][NST], vo1[B_PER][NST];
  int a_at[A_PER], b_at[NCH];                                                       // element offsets inside an LDS buffer
#pragma unroll
  for (int u = 0; u < A_PER; ++u) {
    const int idx = tid + u * THREADS;
    const int row = idx / (TN / 8), cc = idx % (TN / 8);
    va[u] = n0 + 8 * cc < N_out ? 2u * ((uint32_t)row * (uint32_t)ldy + (uint32_t)n0 + 8u * cc) : NOWHERE;
    a_at[u] = row * AP + 8 * cc;
  }
#pragma unroll
  for (int u = 0; u < B_PER; ++u) {
    const int idx = item0 + u * THREADS;
    const int row = idx / CPR, cc = idx % CPR;
    if (SRC == 0) {
      const int c = (int)(j0 / 8) + cc;
      vb[u] = (uint32_t)row * b_pitch + 8u * c;
#pragma unroll
      for (int i = 0; i < NST; ++i) {
        vs[u][i] = 2u * ((uint32_t)row * gpr + (uint32_t)(((seg0 + i) * CPS + c) >> ca.chunk_to_group_shift));
        vo0[u][i] = co.has0[i] ? (uint32_t)row * kk2 + co.vb[i] : NOWHERE;
        vo1[u][i] = co.has1[i] ? (uint32_t)row * kk2 + co.vb[i] + 2u : NOWHERE;
        b_at[u * NST + i] = row * BP + (seg0 + i) * HS + 8 * cc;
      }
    } else {
      vb[u] = (uint32_t)row * b_pitch + 2u * ((uint32_t)j0 + 8u * cc);
      b_at[u] = row * BP + 8 * cc;
    }
  }
  // Chunks with more than two outlier channels are rare, but one of them must not slow the launch down: the third
  // and fourth outlier value of ONE such chunk per thread are requested like everything else (in the stage before
  // they are needed; their cache line arrived with the first two) and written over the decoded chunk in LDS.  What
  // that does not cover (a fifth value, a second such chunk in a thread, 8-bit codes, whose register budget is
  // spent) takes patch_more() below; both conditions are wave-uniform.
  constexpr bool FASTX = SRC == 0 && BITS != 8;
  constexpr int UROW = (THREADS / CPR) * BP;               // elements between a thread's chunks u and u + 1 in an LDS buffer
  bool hasx = false, has4 = false, slow = false;
  int xat2 = 0, xat3 = 0;                                  // LDS element offsets (chunk u = 0) of the two values
  uint32_t vx2 = NOWHERE, vx3 = NOWHERE;                   // their byte offsets in vals, token row 0 of the stage
  if (SRC == 0) {
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int n = __popc(co.m8[i]);
      if (n > 2) {
        if (FASTX && !hasx) {
          hasx = true;
          uint32_t m = co.m8[i];
          m &= m - 1; m &= m - 1;
          xat2 = b_at[i] + (__ffs(m) - 1);
          vx2 = (uint32_t)((item0 / CPR) * kk2) + co.vb[i] + 4u;
          m &= m - 1;
          has4 = m != 0;
          if (has4) { xat3 = b_at[i] + (__ffs(m) - 1); vx3 = vx2 + 2u; }
          slow = slow || n > 4;
        } else {
          slow = true;
        }
      }
    }
  }
  const bool slow_any = __ballot(slow) != 0;
  const BufferRsrc rs_x = make_rsrc(SRC == 0 && ca.k ? vals + m_begin * (int64_t)ca.k : nullptr,
                                    __builtin_amdgcn_readfirstlane((uint32_t)(m_end - m_begin) * kk2));
  // One resource per operand, from the workgroup's first token to the end of its token range; the stage being
  // requested is selected through the scalar offset of the load (the hardware checks the sum of the lane's offset and
  // the scalar one against the size, so a stage past the end reads zeros), which advances by one scalar add per
  // operand and stage.  (Renewing the four resources every stage - a 64-bit add, the remaining length times the pitch
  // and three moves into scalar registers each - was a twelfth of the stage's issue time.)
  const int left0 = (int)(m_end - m_begin);
  const BufferRsrc rs_a = make_rsrc(dy + m_begin * ldy, (uint32_t)left0 * a_pitch);
  const BufferRsrc rs_b = make_rsrc(reinterpret_cast<const char*>(stored) + m_begin * (int64_t)b_pitch,
                                    __builtin_amdgcn_readfirstlane((uint32_t)left0 * b_pitch));
  const BufferRsrc rs_s = make_rsrc(SRC == 0 ? scales + m_begin * (int64_t)gpr : nullptr, SRC == 0 ? (uint32_t)left0 * 2u * gpr : 0u);
  const BufferRsrc rs_o = make_rsrc(SRC == 0 && ca.k ? vals + m_begin * (int64_t)ca.k : nullptr,
                                    __builtin_amdgcn_readfirstlane((uint32_t)left0 * kk2));
  uint32_t so_a = 0, so_b = 0, so_s = 0, so_o = 0;                                  // byte offsets of the stage to request next
  auto advance = [&](int part) __attribute__((always_inline)) {                     // four parts, one operand each
    if (part == 0) so_a += WK * a_pitch;
    else if (part == 1) so_b += WK * b_pitch;
    else if (part == 2 && SRC == 0) so_s += WK * 2u * gpr;
    else if (part == 3 && SRC == 0) so_o += WK * kk2;
    asm volatile("" : "+s"(so_a), "+s"(so_b), "+s"(so_s), "+s"(so_o));              // (in the slot it is written in, in scalar registers)
  };
  // The requests of a stage, numbered: codes and scales (decoded first) before dY and the outlier values.
  constexpr int NLOAD = A_PER + (SRC == 0 ? B_PER * (1 + 3 * NST) : B_PER);
  auto request = [&](Regs& R, int j) __attribute__((always_inline)) {
    if (SRC != 0) {
      if (j < B_PER) R.b[j] = load_b128(rs_b, vb[j], so_b);
      else R.a[j - B_PER] = load_b128(rs_a, va[j - B_PER], so_a);
    } else if (j < B_PER) {
      const uint2 pk = load_b64(rs_b, vb[j], so_b);
      R.b[j] = make_uint4(pk.x, pk.y, 0, 0);
    } else if (j < B_PER + NCH) {
      const int c = j - B_PER;
      R.s[c / NST][c % NST] = load_b16(rs_s, vs[c / NST][c % NST], so_s);
    } else if (j < B_PER + NCH + A_PER) {
      const int u = j - B_PER - NCH;
      R.a[u] = load_b128(rs_a, va[u], so_a);
    } else {
      const int q = j - B_PER - NCH - A_PER, c = q >> 1;
      if (q & 1) R.o1[c / NST][c % NST] = load_b16(rs_o, vo1[c / NST][c % NST], so_o);
      else R.o0[c / NST][c % NST] = load_b16(rs_o, vo0[c / NST][c % NST], so_o);
    }
  };
  auto request_all = [&](Regs& R) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) request(R, j);
#pragma unroll
    for (int part = 0; part < 4; ++part) advance(part);
  };
  // Chunks with more than two outlier channels (rare; the flag is the same for the whole wave): the remaining values
  // are written over the decoded chunk in LDS, element by element, after the chunk itself.
  auto patch_more = [&](uint16_t* Bb, int64_t mb) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      const int idx = item0 + u * THREADS;
      const int row = idx / CPR, cc = idx % CPR;
      if (mb + row < m_end) {
        const uint16_t* vrow = vals + (mb + row) * ca.k;
#pragma unroll
        for (int i = 0; i < NST; ++i) {
          const uint32_t p = ca.plan[(seg0 + i) * CPS + (int)(j0 / 8) + cc];
          uint32_t m = p & 0xFFu;
          m &= m - 1; m &= m - 1;                                       // the first two are in place already
          int at = (int)(p >> 16) + 2;
          while (m != 0) {
            Bb[b_at[u * NST + i] + (__ffs(m) - 1)] = vrow[at++];
            m &= m - 1;
          }
        }
      }
    }
  };
  // decode one stage of registers (tokens mb ..) into an LDS buffer all at once (before the loop)
  auto stash = [&](uint16_t* Ab, uint16_t* Bb, const Regs& R, int64_t mb) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < A_PER; ++u) *reinterpret_cast<uint4*>(&Ab[a_at[u]]) = R.a[u];
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      if (SRC == 0) {
#pragma unroll
        for (int i = 0; i < NST; ++i)
          *reinterpret_cast<uint4*>(&Bb[b_at[u * NST + i]]) =
              co.splice_value(i, dequant8_fast<BITS>(R.b[u].x, R.b[u].y, seg0 + i, bf_to_f((uint16_t)R.s[u][i])), R.o0[u][i], R.o1[u][i]);
      } else {
        *reinterpret_cast<uint4*>(&Bb[b_at[u]]) = R.b[u];
      }
    }
    if (SRC == 0 && co.more_pairs) patch_more(Bb, mb);
  };
  bf16x8_t fa0[4], fb0[4], fa1[4], fb1[4];                    // operand fragments of the stage's first / second 16 tokens
  // fragment q of 8 of a 16-token half: the x fragment of the first MFMAs, the four dY fragments, the other three of x
  auto read_frag = [&](const uint16_t* Ab, const uint16_t* Bb, int kk, int q, bf16x8_t (&fa)[4], bf16x8_t (&fb)[4]) __attribute__((always_inline)) {
    if (q == 0) fb[0] = frag32(Bb, BP, wh, kk);
    else if (q <= 4) fa[q - 1] = frag32(Ab, AP, wn + 32 * (q - 1), kk);
    else fb[q - 4] = frag32(Bb, BP, wh + 32 * (q - 4), kk);
  };
  // One stage: the MFMAs on LDS buffer B; the register set Rd (stage s+1, tokens m1 ..) goes to buffer B+1 on the
  // way and the set Rf is requested anew (stage s+3).
  // What the decode of a stage needs before its first piece - the code bytes of each chunk isolated, its scale as a
  // float and the offset term - is prepared in the last eight slots of the stage before (they are the lightest), as
  // are the requests for the further outlier values of a crowded chunk; both live across the stage boundary.
  constexpr uint32_t REP = (BITS == 8) ? 0x80808080u : Q<BITS>::CODE_MASK * 0x01010101u;
  constexpr float OFFV = (BITS == 8) ? 128.f : (float)Q<BITS>::OFF;
  uint32_t cw[NCH][2];
  float sc[NCH], ns[NCH];
  uint32_t xv2[B_PER], xv3[B_PER];
  auto prepare_codes = [&](const Regs& R, int c) __attribute__((always_inline)) {
    const int u = c / NST, i = c % NST;
    cw[c][0] = (BITS == 8) ? R.b[u].x ^ REP : (R.b[u].x >> ((seg0 + i) * BITS)) & REP;
    cw[c][1] = (BITS == 8) ? R.b[u].y ^ REP : (R.b[u].y >> ((seg0 + i) * BITS)) & REP;
    asm volatile("" : "+v"(cw[c][0]), "+v"(cw[c][1]));                  // (keeps the byte-wise conversions of the pieces)
  };
  auto prepare_scale = [&](const Regs& R, int c) __attribute__((always_inline)) {
    sc[c] = bf_to_f((uint16_t)R.s[c / NST][c % NST]);
    ns[c] = -OFFV * sc[c];
  };
  auto request_extras = [&](int64_t mb, int which) __attribute__((always_inline)) {   // (lanes without a crowded chunk ask for nothing)
    const uint32_t xoff = (uint32_t)(mb - m_begin) * kk2;
#pragma unroll
    for (int u = 0; u < B_PER; ++u) {
      if (which == 0) xv2[u] = load_b16(rs_x, vx2 + xoff + (uint32_t)(u * (THREADS / CPR)) * kk2);
      else xv3[u] = load_b16(rs_x, vx3 + xoff + (uint32_t)(u * (THREADS / CPR)) * kk2);
    }
  };
  // One wait per group of registers instead of one per use: naming them all in an empty asm makes the compiler wait
  // for the last of them here, and the uses that follow need no wait of their own.
  auto arrived_a = [&](Regs& R) __attribute__((always_inline)) {
    asm volatile("" : "+v"(R.a[0].x), "+v"(R.a[1].x), "+v"(R.a[2].x), "+v"(R.a[3].x));   // (one word stands for its load)
  };
  auto arrived_frags = [&](bf16x8_t (&fa)[4], bf16x8_t (&fb)[4]) __attribute__((always_inline)) {
    asm volatile("" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]));
    asm volatile("" : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
  };
  // Rd: decoded and written to LDS in this stage (stage s+1); Rf: requested anew (stage s+3); Rn: decoded in the next
  // stage (stage s+2; its codes and scales are prepared at the end of this one)
  auto stage = [&](auto bno, Regs& Rd, Regs& Rf, const Regs& Rn, int64_t m1) __attribute__((always_inline)) {
    constexpr int B = decltype(bno)::value, NB = (B + 1) % NBUF;
    uint32_t res[NCH][4];
    auto slot = [&](auto tno) __attribute__((always_inline)) {
      constexpr int t = decltype(tno)::value;
      __builtin_amdgcn_sched_barrier(0);
      {
        constexpr int a = t & 3, b = (t >> 2) & 3;
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t < 16 ? fa0[a] : fa1[a], t < 16 ? fb0[b] : fb1[b], acc[a][b], 0, 0, 0);
      }
      if constexpr (t < 8) read_frag(HYC_AS(B), HYC_BS(B), 16, t, fa1, fb1);
      if constexpr (SRC == 0 && t < 16) {                               // two elements of chunk c of stage s+1
        constexpr int c = t >> 2, w = t & 3;
        const uint32_t src = cw[c][w >> 1];
        float c0, c1;
        if constexpr (BITS <= 4) {                                      // both codes of the half-word in one conversion
          const floatx2_t p = (w & 1) ? small_bytes_to_float<true>(src) : small_bytes_to_float<false>(src);
          c0 = p.x; c1 = p.y;
        } else {
          c0 = (float)((src >> (16 * (w & 1))) & 0xFFu); c1 = (float)((src >> (16 * (w & 1) + 8)) & 0xFFu);
        }
        res[c][w] = pack_bf16(__builtin_fmaf(c0, sc[c], ns[c]), __builtin_fmaf(c1, sc[c], ns[c]));
      }
      if constexpr (t >= 8 && t < 16) {
        constexpr int j0_ = (t - 8) * NLOAD / 8, j1_ = (t - 7) * NLOAD / 8;
        for_each_slot([&](auto jno) __attribute__((always_inline)) { request(Rf, j0_ + decltype(jno)::value); },
                      std::make_integer_sequence<int, j1_ - j0_>{});
      }
      if constexpr (t == 16) {
        arrived_a(Rd);
        arrived_frags(fa1, fb1);
      }
      if constexpr (t >= 16 && t < 20) {
        *reinterpret_cast<uint4*>(&HYC_AS(NB)[a_at[t - 16]]) = Rd.a[t - 16];
        advance(t - 16);
      }
      if constexpr (t >= 20 && t < 24) {
        constexpr int c = t - 20, u = c / NST, i = c % NST;
        if constexpr (SRC == 0)
          *reinterpret_cast<uint4*>(&HYC_BS(NB)[b_at[c]]) =
              co.splice_value(i, make_uint4(res[c][0], res[c][1], res[c][2], res[c][3]), Rd.o0[u][i], Rd.o1[u][i]);
        else
          *reinterpret_cast<uint4*>(&HYC_BS(NB)[b_at[c]]) = Rd.b[c];
        if constexpr (t == 23 && SRC == 0) {
          if (co.more_pairs) {
            if (FASTX && hasx) {
#pragma unroll
              for (int u = 0; u < B_PER; ++u) {
                HYC_BS(NB)[xat2 + u * UROW] = (uint16_t)xv2[u];
                if (has4) HYC_BS(NB)[xat3 + u * UROW] = (uint16_t)xv3[u];
              }
            }
            if (!FASTX || slow_any) patch_more(HYC_BS(NB), m1);
          }
        }
      }
      if constexpr (t == 24) __syncthreads();                           // buffer NB is complete, buffer B read for the last time
      if constexpr (t >= 24) read_frag(HYC_AS(NB), HYC_BS(NB), 0, t - 24, fa0, fb0);
      if constexpr (SRC == 0 && t >= 24) {                              // for the next stage's decode
        if constexpr ((t & 1) == 0) prepare_codes(Rn, (t - 24) >> 1); else prepare_scale(Rn, (t - 24) >> 1);
        if constexpr (FASTX && (t == 26 || t == 27)) request_extras(m1 + WK, t - 26);
      }
    };
    for_each_slot(slot, std::make_integer_sequence<int, 32>{});
    __builtin_amdgcn_sched_barrier(0);
  };

  if (m_begin < m_end) {
    Regs R0, R1, R2;
    const int64_t nstages = (m_end - m_begin + WK - 1) / WK;
    request_all(R0);
    request_all(R1);
    request_all(R2);
    stash(HYC_AS(0), HYC_BS(0), R0, m_begin);
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 8; ++q) read_frag(HYC_AS(0), HYC_BS(0), 0, q, fa0, fb0);
    int64_t m1 = m_begin + WK;
    if (SRC == 0) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) { prepare_codes(R1, c); prepare_scale(R1, c); }
      if (FASTX) { request_extras(m1, 0); request_extras(m1, 1); }
    }
    for (int64_t s = 0; s < nstages; s += 3) {                         // a stage past the end holds zeros
      stage(StageNo<0>{}, R1, R0, R2, m1);
      stage(StageNo<1>{}, R2, R1, R0, m1 + WK);
      stage(StageNo<2>{}, R0, R2, R1, m1 + 2 * WK);
      m1 += 3 * WK;
    }
  }
#undef HYC_AS
#undef HYC_BS

  // ---- epilogue.  A lane holds column (lane mod 32), rows 8*(v/4) + 4*(lane/32) + (v mod 4) of each 32x32 tile.  The
  // wave turns 32 rows x 128 columns at a time around in a private piece of LDS so that every lane stores eight
  // neighbouring columns (16 bytes of bf16, 32 of fp32) and a row leaves as one contiguous run. ----
  constexpr int EPP = 128 + 4;                               // floats per staged row
  static_assert(4 * 32 * EPP * 4 <= (int)sizeof(lds), "epilogue staging");
  __syncthreads();                                           // the last fragments have been read
  float* ep = reinterpret_cast<float*>(lds) + wave * (32 * EPP);
  const int er = lane >> 4, ec = 8 * (lane & 15);
  const int hl = wh + ec;                                    // first of the lane's columns inside the tile
  const int64_t h = (int64_t)(hl / HS) * SEG + j0 + (hl % HS);
#pragma unroll
  for (int a = 0; a < 4; ++a) {
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) ep[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * EPP + 32 * b + (lane & 31)] = acc[a][b][v];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // (one wave: LDS keeps its order, the compiler must too)
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int r = 4 * p + er;
      const int64_t n = n0 + wn + 32 * a + r;
      float4 lo = *reinterpret_cast<const float4*>(&ep[r * EPP + ec]);
      float4 hi = *reinterpret_cast<const float4*>(&ep[r * EPP + ec + 4]);
      if (n < N_out) {
        if (partial != nullptr) {
          float4* o = reinterpret_cast<float4*>(partial + ((int64_t)blockIdx.z * N_out + n) * H + h);
          o[0] = lo; o[1] = hi;
        } else if (out_f32) {
          float4* o = reinterpret_cast<float4*>(static_cast<float*>(out) + n * H + h);
          float4 p0 = make_float4(0.f, 0.f, 0.f, 0.f), p1 = p0;
          if (beta != 0.f) { p0 = o[0]; p1 = o[1]; }
          o[0] = make_float4(alpha * lo.x + beta * p0.x, alpha * lo.y + beta * p0.y, alpha * lo.z + beta * p0.z, alpha * lo.w + beta * p0.w);
          o[1] = make_float4(alpha * hi.x + beta * p1.x, alpha * hi.y + beta * p1.y, alpha * hi.z + beta * p1.z, alpha * hi.w + beta * p1.w);
        } else {
          uint4* o = reinterpret_cast<uint4*>(static_cast<uint16_t*>(out) + n * H + h);
          uint4 q = make_uint4(0, 0, 0, 0);
          if (beta != 0.f) q = *o;
          auto mix = [&](float x0, float x1, uint32_t old) __attribute__((always_inline)) {
            return pack_bf16(alpha * x0 + beta * bf_to_f((uint16_t)(old & 0xFFFFu)), alpha * x1 + beta * bf_to_f((uint16_t)(old >> 16)));
          };
          *o = make_uint4(mix(lo.x, lo.y, q.x), mix(lo.z, lo.w, q.y), mix(hi.x, hi.y, q.z), mix(hi.z, hi.w, q.w));
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

// out = alpha * sum_z partial[z] + beta * out, splits added in increasing z
__global__ void __launch_bounds__(256)
k_gradw_finish(const float* __restrict__ partial, int splits, int64_t total, float alpha, float beta,
               void* __restrict__ out, int out_f32) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  float s = 0.f;
  int z = 0;
  for (; z + 8 <= splits; z += 8) {                       // eight loads in flight, added in increasing z
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) t[u] = partial[(int64_t)(z + u) * total + i];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += t[u];
  }
  for (; z < splits; ++z) s += partial[(int64_t)z * total + i];
  if (out_f32) {
    float* o = static_cast<float*>(out) + i;
    *o = (beta != 0.f) ? alpha * s + beta * *o : alpha * s;
  } else {
    uint16_t* o = static_cast<uint16_t*>(out) + i;
    *o = f_to_bf((beta != 0.f) ? alpha * s + beta * bf_to_f(*o) : alpha * s);
  }
}

// how many token splits to use: fill the chip when the output grid alone cannot
static int choose_splits(int64_t M, int64_t tiles) {
  if (tiles >= 512) return 1;
  int64_t s = (1024 + tiles - 1) / tiles;
  const int64_t max_by_tokens = (M + 4 * GK - 1) / (4 * GK);      // at least 4 stages per split
  if (s > max_by_tokens) s = max_by_tokens;
  if (s < 1) s = 1;
  if (s > 64) s = 64;
  return (int)s;
}

// ... for the 256 x 256 tiles of k_gradw_big, one workgroup per CU at a time.  A split costs a partial result written
// and read again: 8 bytes per output element at about 4 TB/s against 2*M flop per element at about 1.1 PFLOP/s, i.e.
// 1100 / M of the product's own time per split; the rounds of workgroups cost 1 / (filled share of the last round).
static int choose_splits_big(int64_t M, int64_t tiles) {
  const int64_t cus = 256;
  const int64_t max_by_tokens = std::max<int64_t>(1, M / (8 * WK));   // at least 8 stages per split
  int best = 1;
  double best_cost = 0.0;
  for (int64_t s = 1; s <= 16 && s <= max_by_tokens; ++s) {
    const int64_t wgs = tiles * s;
    const double rounds = (double)(((wgs + cus - 1) / cus) * cus) / (double)wgs;
    const double cost = rounds + (s > 1 ? (double)s * 1100.0 / (double)M : 0.0);
    if (s == 1 || cost < best_cost - 1e-9) { best_cost = cost; best = (int)s; }
  }
  return best;
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int64_t hyc_gradw_workspace_bytes(int64_t M, int64_t N_out, int64_t H) {
  if (M <= 0 || N_out <= 0 || H <= 0) return 0;
  const int BN = N_out <= 32 ? 32 : 128;
  const int64_t tiles = ((N_out + BN - 1) / BN) * (H / GH);
  int splits = choose_splits(M, tiles);                   // dense source
  if (N_out >= 2 * WN && H % GH == 0)                     // 256 x 256 tiles
    splits = std::max(splits, choose_splits_big(M, ((N_out + 2 * WN - 1) / (2 * WN)) * ((H + WH - 1) / WH)));
  if (N_out <= DIRECT_MAX_N) {                            // channel-compressed source, few output rows
    const int ds = direct_splits_max(M, N_out, H);
    if (ds > splits) splits = ds;
  }
  return splits > 1 ? (int64_t)splits * N_out * H * 4 : 0;
}

int hyc_gradw_gemm(const void* dy, int64_t ldy, const void* stored, const void* vals, const void* scales, int64_t M,
                   int64_t N_out, int64_t H, const hyc_desc* d, float alpha, float beta, void* out, int32_t out_dtype,
                   void* workspace, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_gradw_gemm: null descriptor");
  if (M < 0 || N_out <= 0) return fail(HYC_EINVAL, "hyc_gradw_gemm: M=%lld N_out=%lld", (long long)M, (long long)N_out);
  if (out_dtype != HYC_DTYPE_BF16 && out_dtype != HYC_DTYPE_F32) return fail(HYC_EINVAL, "hyc_gradw_gemm: out_dtype=%d", out_dtype);
  if (d->mode == HYC_MODE_THRESHOLD)
    return fail(HYC_ENOTSUP, "hyc_gradw_gemm: threshold-mode activations are decompressed first (hyc_decompress) and passed with HYC_MODE_DENSE");
  if (d->mode != HYC_MODE_CHANNEL && d->mode != HYC_MODE_DENSE) return fail(HYC_EINVAL, "hyc_gradw_gemm: mode=%d", d->mode);
  if (N_out % 8 != 0 || ldy % 8 != 0 || ldy < N_out)
    return fail(HYC_ENOTSUP, "hyc_gradw_gemm: N_out=%lld and ldy=%lld must be multiples of 8, ldy >= N_out", (long long)N_out, (long long)ldy);
  RowGeom g;
  ChanArgs ca = {};
  int lpg = 16, rc;
  const bool chan = d->mode == HYC_MODE_CHANNEL;
  if (chan) {
    if ((rc = row_geom(H, d->bits, &g))) return rc;
    if ((rc = make_chan_args(d, g, &ca, &lpg))) return rc;
    const int hs = GH / g.nseg;
    if (N_out > DIRECT_MAX_N && g.seg % hs != 0)
      return fail(HYC_ENOTSUP, "hyc_gradw_gemm: H*bits/8=%lld must be a multiple of %d when N_out > %d", (long long)g.seg, hs, (int)DIRECT_MAX_N);
  } else {
    if (H <= 0 || H % GH != 0) return fail(HYC_ENOTSUP, "hyc_gradw_gemm: dense H=%lld must be a multiple of %d", (long long)H, GH);
    g.cps = (int)(H / 8);
  }
  if (!out) return fail(HYC_EFAULT, "hyc_gradw_gemm: null out");
  hipStream_t st = begin_launch(stream);
  if (chan && N_out <= DIRECT_MAX_N) {
    if (M > 0 && (!dy || !stored || !scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_gradw_gemm: null buffer");
    if (M > 0 && !aligned8(stored)) return fail(HYC_EINVAL, "hyc_gradw_gemm: stored must be 8-byte aligned");
    const DirectPlan pl = direct_plan(d->bits, N_out);
    const int c_tiles = (g.cps + 15) / 16, o_tiles = (d->k + 15) / 16;
    const int y_tiles = (g.nseg / pl.spt) * c_tiles + o_tiles;
    const int x_tiles = (int)direct_x_tiles(N_out);
    const int nw = direct_waves(M, (int64_t)y_tiles * x_tiles, pl.per_cu);
    const int splits = M > 0 ? direct_splits(M, (int64_t)y_tiles * x_tiles, nw, pl.per_cu) : 1;
    if (splits > 1 && !workspace) return fail(HYC_EFAULT, "hyc_gradw_gemm: workspace of hyc_gradw_workspace_bytes() bytes required");
    if (splits > 1 && !aligned16(workspace)) return fail(HYC_EINVAL, "hyc_gradw_gemm: workspace must be 16-byte aligned");
    int64_t tps = (M + splits - 1) / splits;
    tps = ((tps + DK - 1) / DK) * DK;
    if (tps < DK) tps = DK;
    float* partial = splits > 1 ? static_cast<float*>(workspace) : nullptr;
    const int nt = N_out <= 16 ? 1 : 2;
    const dim3 grid((unsigned)x_tiles, (unsigned)y_tiles, (unsigned)splits);
    const int of32 = out_dtype == HYC_DTYPE_F32;
    DirectArgs da = {static_cast<const uint16_t*>(dy), ldy, M, N_out, H, static_cast<const uint8_t*>(stored),
                     static_cast<const uint16_t*>(vals), static_cast<const uint16_t*>(scales), ca, g.cps, c_tiles, tps,
                     alpha, beta, out, of32, partial};
#define HYC_DIRECT_K(B_, N_, S_)                                                                               \
  do {                                                                                                         \
    if (nw == 8) hipLaunchKernelGGL((k_gradw_direct<B_, N_, S_, 8>), grid, dim3(512), 0, st, da);              \
    else hipLaunchKernelGGL((k_gradw_direct<B_, N_, S_, 4>), grid, dim3(256), 0, st, da);                      \
  } while (0)
#define HYC_DIRECT(B_) do { if (nt == 1) HYC_DIRECT_K(B_, 1, (B_ < 8 ? 2 : 1)); else HYC_DIRECT_K(B_, 2, 1); } while (0)   /* direct_plan() */
    switch (d->bits) {
      case 1: HYC_DIRECT(1); break;
      case 2: HYC_DIRECT(2); break;
      case 4: HYC_DIRECT(4); break;
      default: HYC_DIRECT(8); break;
    }
#undef HYC_DIRECT_K
#undef HYC_DIRECT
    if ((rc = check_launch("hyc_gradw_gemm"))) return rc;
    if (splits > 1) {
      const int64_t total = N_out * H;
      hipLaunchKernelGGL(k_gradw_finish, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, partial, splits, total,
                         alpha, beta, out, of32);
      return check_launch("hyc_gradw_gemm (finish)");
    }
    return HYC_OK;
  }
  const int BN = N_out <= 32 ? 32 : 128;
  const int64_t n_tiles = (N_out + BN - 1) / BN, h_tiles = H / GH;
  if (M > 0 && (!dy || !stored)) return fail(HYC_EFAULT, "hyc_gradw_gemm: null buffer");
  // wide tiles (256 columns) when the output is large and the tile grid fits the packing
  // (the channel scheme has the 256-feature form only)
  const bool wide = chan ? (N_out >= 2 * WN && g.seg % (WH / g.nseg) == 0) : (N_out >= WN && H % WH == 0);
  // 256 features per workgroup (four waves of 128 x 128) from 256 output features on, else 128 (dense only); a tile
  // grid below the CU count is made up with token splits
  const int wnt = !wide ? 0 : chan || N_out >= 2 * WN ? 2 * WN : WN;
  const int splits = M <= 0 ? 1 : wnt == 2 * WN ? choose_splits_big(M, ((N_out + 2 * WN - 1) / (2 * WN)) * (H / WH))
                                                : choose_splits(M, n_tiles * h_tiles);   // (128 x 256 tiles: same value)
  if (chan && M > 0 && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_gradw_gemm: null vals/scales");
  if (M > 0 && (!aligned16(dy) || !aligned8(stored) || (!chan && !aligned16(stored))))
    return fail(HYC_EINVAL, "hyc_gradw_gemm: dy must be 16-byte aligned, stored 8-byte (16 when dense)");
  if (splits > 1 && !workspace) return fail(HYC_EFAULT, "hyc_gradw_gemm: workspace of hyc_gradw_workspace_bytes() bytes required");
  int64_t tps = (M + splits - 1) / splits;
  tps = ((tps + GK - 1) / GK) * GK;
  float* partial = splits > 1 ? static_cast<float*>(workspace) : nullptr;
  const dim3 grid((unsigned)n_tiles, (unsigned)h_tiles, (unsigned)splits);
  const int of32 = out_dtype == HYC_DTYPE_F32;
  // the wide kernel addresses a workgroup's token range with 32-bit offsets: each operand's share must stay under 2 GiB
  const int64_t pitch_max = std::max<int64_t>(std::max<int64_t>(2 * ldy, chan ? g.seg : 2 * H),
                                              chan ? std::max<int64_t>(2 * (H / d->group), 2 * (int64_t)d->k) : 0);
  const bool fits32 = (tps + WK) * pitch_max < ((int64_t)1 << 31);
  if (wide && fits32) {
    const dim3 wgrid((unsigned)((N_out + wnt - 1) / wnt), (unsigned)(H / WH), (unsigned)splits);
#define HYC_WIDE()                                                                                               \
  hipLaunchKernelGGL(k_gradw_wide, wgrid, dim3(2 * WN), 0, st, static_cast<const uint16_t*>(dy), ldy, M, N_out, H, \
                     static_cast<const uint16_t*>(stored), tps, alpha, beta, out, of32, partial)
#define HYC_BIG(B_, S_)                                                                                            \
  hipLaunchKernelGGL((k_gradw_big<B_, S_>), wgrid, dim3(256), 0, st, static_cast<const uint16_t*>(dy), ldy, M,     \
                     N_out, H, static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),          \
                     static_cast<const uint16_t*>(scales), ca, g.cps, tps, alpha, beta, out, of32, partial)
    if (wnt == WN) {
      HYC_WIDE();
    } else if (chan) {
      switch (d->bits) {
        case 1: HYC_BIG(1, 0); break;
        case 2: HYC_BIG(2, 0); break;
        case 4: HYC_BIG(4, 0); break;
        default: HYC_BIG(8, 0); break;
      }
    } else {
      HYC_BIG(4, 2);
    }
#undef HYC_BIG
#undef HYC_WIDE
  } else {
#define HYC_GEMM(B_, S_, N_)                                                                                     \
  hipLaunchKernelGGL((k_gradw<B_, S_, N_>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(dy), ldy, M, N_out, H, \
                     static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                    \
                     static_cast<const uint16_t*>(scales), ca, g.cps, tps, alpha, beta, out, of32, partial)
#define HYC_GEMM_BN(B_, S_) do { if (BN == 128) HYC_GEMM(B_, S_, 128); else HYC_GEMM(B_, S_, 32); } while (0)
  if (chan) {
    switch (d->bits) {
      case 1: HYC_GEMM_BN(1, 0); break;
      case 2: HYC_GEMM_BN(2, 0); break;
      case 4: HYC_GEMM_BN(4, 0); break;
      default: HYC_GEMM_BN(8, 0); break;
    }
  } else {
    HYC_GEMM_BN(4, 2);
  }
#undef HYC_GEMM_BN
#undef HYC_GEMM
  }
  if ((rc = check_launch("hyc_gradw_gemm"))) return rc;
  if (splits > 1) {
    const int64_t total = N_out * H;
    hipLaunchKernelGGL(k_gradw_finish, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, partial, splits, total,
                       alpha, beta, out, of32);
    return check_launch("hyc_gradw_gemm (finish)");
  }
  return HYC_OK;
}

}  // extern "C"
