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

// out = alpha * sum_z partial[z] + beta * out, splits added in increasing z
__global__ void __launch_bounds__(256)
k_gradw_finish(const float* __restrict__ partial, int splits, int64_t total, float alpha, float beta,
               void* __restrict__ out, int out_f32) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  float s = 0.f;
  for (int z = 0; z < splits; ++z) s += partial[(int64_t)z * total + i];
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

}  // namespace hyc

using namespace hyc;

extern "C" {

int64_t hyc_gradw_workspace_bytes(int64_t M, int64_t N_out, int64_t H) {
  if (M <= 0 || N_out <= 0 || H <= 0) return 0;
  const int BN = N_out <= 32 ? 32 : 128;
  const int64_t tiles = ((N_out + BN - 1) / BN) * (H / GH);
  const int splits = choose_splits(M, tiles);
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
    if (g.seg % hs != 0) return fail(HYC_ENOTSUP, "hyc_gradw_gemm: H*bits/8=%lld must be a multiple of %d", (long long)g.seg, hs);
  } else {
    if (H <= 0 || H % GH != 0) return fail(HYC_ENOTSUP, "hyc_gradw_gemm: dense H=%lld must be a multiple of %d", (long long)H, GH);
    g.cps = (int)(H / 8);
  }
  if (!out) return fail(HYC_EFAULT, "hyc_gradw_gemm: null out");
  hipStream_t st = begin_launch(stream);
  const int BN = N_out <= 32 ? 32 : 128;
  const int64_t n_tiles = (N_out + BN - 1) / BN, h_tiles = H / GH;
  const int splits = M > 0 ? choose_splits(M, n_tiles * h_tiles) : 1;
  if (M > 0 && (!dy || !stored)) return fail(HYC_EFAULT, "hyc_gradw_gemm: null buffer");
  if (chan && M > 0 && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_gradw_gemm: null vals/scales");
  if (M > 0 && (!aligned16(dy) || !aligned8(stored) || (!chan && !aligned16(stored))))
    return fail(HYC_EINVAL, "hyc_gradw_gemm: dy must be 16-byte aligned, stored 8-byte (16 when dense)");
  if (splits > 1 && !workspace) return fail(HYC_EFAULT, "hyc_gradw_gemm: workspace of hyc_gradw_workspace_bytes() bytes required");
  int64_t tps = (M + splits - 1) / splits;
  tps = ((tps + GK - 1) / GK) * GK;
  float* partial = splits > 1 ? static_cast<float*>(workspace) : nullptr;
  const dim3 grid((unsigned)n_tiles, (unsigned)h_tiles, (unsigned)splits);
  const int of32 = out_dtype == HYC_DTYPE_F32;
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
