// RMSNorm forward fused with the compression of its input, and RMSNorm backward fused with the
// decompression.  One workgroup per row at a time; the row lives in registers (x is read from HBM once).
#include "abi_util.hpp"
#include "row_kernels.hpp"

namespace hyc {

// 8 weights at `col` as floats; w is bf16 or fp32 (uniform runtime switch)
__device__ __forceinline__ void load_w8(const void* w, bool wf32, int64_t col, float (&o)[8]) {
  if (wf32) {
    const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + col);
    const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + col + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    unpack8(*reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(w) + col), o);
  }
}

// two block-wide sums at once; red holds >= 32 floats
__device__ __forceinline__ void block_sum2(float& a, float& b, float* red) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  if ((threadIdx.x & 63) == 0) { red[wave] = a; red[16 + wave] = b; }
  __syncthreads();
  float ta = 0.f, tb = 0.f;
  for (int i = 0; i < nw; ++i) { ta += red[i]; tb += red[16 + i]; }
  __syncthreads();
  a = ta; b = tb;
}

// ------------------------------------------------------------------------------------------------
// forward: y, rstd, and x compressed.  MODE 0 = channel, 1 = threshold.
// ------------------------------------------------------------------------------------------------
template <int BITS, int ITERS, int MAXT, int MODE>
__global__ void __launch_bounds__(MAXT)
k_rmsnorm_fwd(const uint16_t* __restrict__ x, const void* __restrict__ w, bool wf32, float eps, int64_t M, int64_t H,
              int CPS, ChanArgs ca, int lpg, ThrArgs ta, bool perchan, uint16_t* __restrict__ y,
              float* __restrict__ rstd_out, uint8_t* __restrict__ stored, uint16_t* __restrict__ vals,
              uint16_t* __restrict__ scales, int32_t* __restrict__ row_counts) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ float red[32];
  const int64_t SEG = (int64_t)CPS * 8;
  const float invH = 1.0f / (float)H;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* xr = x + row * H;
    uint4 raw[ITERS][NSEG];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      const bool active = c < CPS;
#pragma unroll
      for (int i = 0; i < NSEG; ++i)
        raw[it][i] = active ? *reinterpret_cast<const uint4*>(xr + i * SEG + 8 * c) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float v[8];
        unpack8(raw[it][i], v);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(v[j], v[j], ss);
      }
    // compress x (independent of rstd)
    float hot = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      const bool active = c < CPS;
      uint32_t lo, hi;
      if (MODE == 0) {
        encode_chan<BITS>(raw[it], active, c, CPS, lpg, ca, vals + row * ca.k, scales + row * ca.groups_per_row, lo, hi);
      } else {
        if (active) {
          hot += (float)(perchan ? encode_thr<BITS, true>(raw[it], c, CPS, H, row % ta.S, ta, lo, hi)
                                 : encode_thr<BITS, false>(raw[it], c, CPS, H, row % ta.S, ta, lo, hi));
        }
      }
      if (active) *reinterpret_cast<uint2*>(stored + row * SEG + 8 * c) = make_uint2(lo, hi);
    }
    block_sum2(ss, hot, red);
    const float rstd = 1.0f / __builtin_sqrtf(ss * invH + eps);
    if (threadIdx.x == 0) {
      rstd_out[row] = rstd;
      if (MODE == 1 && row_counts) row_counts[row] = (int32_t)hot;
    }
    uint16_t* yr = y + row * H;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          const int64_t col = i * SEG + 8 * c;
          float v[8], wv[8];
          unpack8(raw[it][i], v);
          load_w8(w, wf32, col, wv);
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = (v[j] * rstd) * wv[j];
          *reinterpret_cast<uint4*>(yr + col) = pack8(v);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// backward.  SRC 0 = channel-compressed x, 2 = dense bf16 x_hat.  Rows [blockIdx.x*rpb, +rpb).
// ------------------------------------------------------------------------------------------------
template <int BITS, int ITERS, int MAXT, int SRC>
__global__ void __launch_bounds__(MAXT)
k_rmsnorm_bwd(const uint16_t* __restrict__ dy, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
              const uint16_t* __restrict__ scales, const void* __restrict__ w, bool wf32,
              const float* __restrict__ rstd, int64_t M, int64_t H, int CPS, int rows_per_block, ChanArgs ca,
              bool quirk, uint16_t* __restrict__ dx, float* __restrict__ dw_partials) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ float red[32];
  const int64_t SEG = (int64_t)CPS * 8;
  const float invH = 1.0f / (float)H;
  float wv[ITERS][NSEG][8], acc[ITERS][NSEG][8];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = it * blockDim.x + threadIdx.x;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      if (c < CPS) load_w8(w, wf32, i * SEG + 8 * c, wv[it][i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) { acc[it][i][j] = 0.f; if (c >= CPS) wv[it][i][j] = 0.f; }
    }
  }
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < M ? r0 + rows_per_block : M;
  for (int64_t row = r0; row < r1; ++row) {
    const float rs = rstd[row];
    float xn[ITERS][NSEG][8], wdy[ITERS][NSEG][8];
    float p1 = 0.f, p2 = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      const bool active = c < CPS;
      uint2 pk = make_uint2(0, 0);
      if (SRC == 0 && active) pk = *reinterpret_cast<const uint2*>(stored + row * SEG + 8 * c);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        const int64_t col = i * SEG + 8 * c;
        float g[8];
        if (active) {
          unpack8(*reinterpret_cast<const uint4*>(dy + row * H + col), g);
          if (SRC == 0) {
            decode_chan<BITS>(pk.x, pk.y, i, c, CPS, ca, vals + row * ca.k, scales + row * ca.groups_per_row, xn[it][i]);
          } else {
            unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(stored) + row * H + col), xn[it][i]);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) { g[j] = 0.f; xn[it][i][j] = 0.f; }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float n = xn[it][i][j] * rs;
          const float t = wv[it][i][j] * g[j];
          xn[it][i][j] = n;
          wdy[it][i][j] = t;
          p1 = __builtin_fmaf(n, t, p1);
          p2 += t;
          acc[it][i][j] = __builtin_fmaf(g[j], n, acc[it][i][j]);
        }
      }
    }
    block_sum2(p1, p2, red);
    const float c1 = p1 * invH;
    const float c2 = quirk ? p2 * invH : 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          float o[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = (wdy[it][i][j] - (xn[it][i][j] * c1 + c2)) * rs;
          *reinterpret_cast<uint4*>(dx + row * H + i * SEG + 8 * c) = pack8(o);
        }
      }
    }
  }
  float* pr = dw_partials + (int64_t)blockIdx.x * H;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = it * blockDim.x + threadIdx.x;
    if (c < CPS) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float4* o = reinterpret_cast<float4*>(pr + i * SEG + 8 * c);
        o[0] = make_float4(acc[it][i][0], acc[it][i][1], acc[it][i][2], acc[it][i][3]);
        o[1] = make_float4(acc[it][i][4], acc[it][i][5], acc[it][i][6], acc[it][i][7]);
      }
    }
  }
}

// dw[c] = sum_p partials[p, c] in a fixed order: 32 columns x 8 row lanes per workgroup, each lane sums rows
// p = lane, lane+8, ... and the 8 lane sums are added in lane order.
__global__ void __launch_bounds__(256)
k_colsum(const float* __restrict__ partials, int64_t P, int64_t H, void* __restrict__ dw, bool wf32) {
  __shared__ float part[8][33];
  const int cx = threadIdx.x & 31, lane = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + cx;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (c < H) {
    int64_t p = lane;
    for (; p + 24 < P; p += 32) {
      s0 += partials[p * H + c];
      s1 += partials[(p + 8) * H + c];
      s2 += partials[(p + 16) * H + c];
      s3 += partials[(p + 24) * H + c];
    }
    for (; p < P; p += 8) s0 += partials[p * H + c];
  }
  part[lane][cx] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (lane == 0 && c < H) {
    float s = 0.f;
#pragma unroll
    for (int l = 0; l < 8; ++l) s += part[l][cx];
    if (wf32) static_cast<float*>(dw)[c] = s;
    else static_cast<uint16_t*>(dw)[c] = f_to_bf(s);
  }
}

static inline int64_t bwd_rows_per_block(int64_t M) {
  // about a thousand workgroups, at least four rows each
  int64_t rpb = (M + 1023) / 1024;
  return rpb < 4 ? 4 : rpb;
}

}  // namespace hyc

using namespace hyc;

#define HYC_BITS_ITERS_MAXT(BITS_, ITERS_, THREADS_, ...)                                   \
  do {                                                                                      \
    const int key_ = (BITS_) * 100 + (ITERS_) * 10 + ((THREADS_) > 256 ? 1 : 0);            \
    switch (key_) {                                                                         \
      HYC_CASE_(1, 1, __VA_ARGS__) HYC_CASE_(1, 2, __VA_ARGS__) HYC_CASE_(1, 4, __VA_ARGS__)  \
      HYC_CASE_(2, 1, __VA_ARGS__) HYC_CASE_(2, 2, __VA_ARGS__) HYC_CASE_(2, 4, __VA_ARGS__)  \
      HYC_CASE_(4, 1, __VA_ARGS__) HYC_CASE_(4, 2, __VA_ARGS__) HYC_CASE_(4, 4, __VA_ARGS__)  \
      HYC_CASE_(8, 1, __VA_ARGS__) HYC_CASE_(8, 2, __VA_ARGS__) HYC_CASE_(8, 4, __VA_ARGS__)  \
      default: return fail(HYC_ENOTSUP, "row too long for the fused kernels (bits=%d)", (BITS_)); \
    }                                                                                       \
  } while (0)
#define HYC_CASE_(B_, I_, ...)                                                              \
  case (B_) * 100 + (I_) * 10 + 0: { constexpr int B = B_, IT = I_, MT = 256; __VA_ARGS__; } break;  \
  case (B_) * 100 + (I_) * 10 + 1: { constexpr int B = B_, IT = I_, MT = 1024; __VA_ARGS__; } break;

static inline int round_iters(int iters) { return iters <= 1 ? 1 : iters <= 2 ? 2 : iters <= 4 ? 4 : 99; }

extern "C" {

int64_t hyc_rmsnorm_bwd_partials(int64_t M, int64_t H) {
  (void)H;
  if (M <= 0) return 0;
  const int64_t rpb = bwd_rows_per_block(M);
  return (M + rpb - 1) / rpb;
}

int hyc_rmsnorm_fwd_compress(const void* x, const void* w, int32_t w_dtype, float eps, int64_t M, int64_t H,
                             const hyc_desc* d, void* y, float* rstd, void* stored, void* vals, void* scales,
                             int32_t* row_counts, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_rmsnorm_fwd_compress: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_rmsnorm_fwd_compress: M=%lld", (long long)M);
  if (w_dtype != HYC_DTYPE_BF16 && w_dtype != HYC_DTYPE_F32) return fail(HYC_EINVAL, "hyc_rmsnorm_fwd_compress: w_dtype=%d", w_dtype);
  RowGeom g;
  int rc = row_geom(H, d->bits, &g);
  if (rc) return rc;
  ChanArgs ca = {}; ThrArgs ta = {}; int lpg = 16; bool perchan = false;
  if (d->mode == HYC_MODE_CHANNEL) { if ((rc = make_chan_args(d, g, &ca, &lpg))) return rc; }
  else if (d->mode == HYC_MODE_THRESHOLD) { if ((rc = make_thr_args(d, g, &ta, &perchan))) return rc; }
  else return fail(HYC_EINVAL, "hyc_rmsnorm_fwd_compress: mode=%d", d->mode);
  if (M == 0) return HYC_OK;
  if (!x || !w || !y || !rstd || !stored) return fail(HYC_EFAULT, "hyc_rmsnorm_fwd_compress: null buffer");
  if (d->mode == HYC_MODE_CHANNEL && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_rmsnorm_fwd_compress: null vals/scales");
  if (!aligned16(x) || !aligned16(y) || !aligned16(w) || !aligned8(stored))
    return fail(HYC_EINVAL, "hyc_rmsnorm_fwd_compress: x, y, w must be 16-byte and stored 8-byte aligned");
  const bool wf32 = w_dtype == HYC_DTYPE_F32;
  const int64_t cap = 256 * (g.threads >= 512 ? 3 : 8);
  const int grid = (int)(M < cap ? M : cap);
  hipStream_t st = begin_launch(stream);
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  if (d->mode == HYC_MODE_CHANNEL) {
    HYC_BITS_ITERS_MAXT(d->bits, round_iters(g.iters), g.threads,
      hipLaunchKernelGGL((k_rmsnorm_fwd<B, IT, MT, 0>), dim3(grid), dim3(g.threads), 0, st, xp, w, wf32, eps, M, H, g.cps,
                         ca, lpg, ta, perchan, static_cast<uint16_t*>(y), rstd, static_cast<uint8_t*>(stored),
                         static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales), row_counts));
  } else {
    HYC_BITS_ITERS_MAXT(d->bits, round_iters(g.iters), g.threads,
      hipLaunchKernelGGL((k_rmsnorm_fwd<B, IT, MT, 1>), dim3(grid), dim3(g.threads), 0, st, xp, w, wf32, eps, M, H, g.cps,
                         ca, lpg, ta, perchan, static_cast<uint16_t*>(y), rstd, static_cast<uint8_t*>(stored),
                         static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales), row_counts));
  }
  return check_launch("hyc_rmsnorm_fwd_compress");
}

int hyc_rmsnorm_bwd(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                    int32_t w_dtype, const float* rstd, int64_t M, int64_t H, const hyc_desc* d, int32_t c2_quirk,
                    void* dx, float* dw_partials, void* dw, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_rmsnorm_bwd: M=%lld", (long long)M);
  if (w_dtype != HYC_DTYPE_BF16 && w_dtype != HYC_DTYPE_F32) return fail(HYC_EINVAL, "hyc_rmsnorm_bwd: w_dtype=%d", w_dtype);
  if (d->mode == HYC_MODE_THRESHOLD)
    return fail(HYC_ENOTSUP, "hyc_rmsnorm_bwd: threshold-mode activations are decompressed first (hyc_decompress) and passed with HYC_MODE_DENSE");
  if (d->mode != HYC_MODE_CHANNEL && d->mode != HYC_MODE_DENSE) return fail(HYC_EINVAL, "hyc_rmsnorm_bwd: mode=%d", d->mode);
  RowGeom g;
  int rc = row_geom(H, d->bits, &g);
  if (rc) return rc;
  ChanArgs ca = {}; int lpg = 16;
  if (d->mode == HYC_MODE_CHANNEL && (rc = make_chan_args(d, g, &ca, &lpg))) return rc;
  if (!dw) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null dw");
  hipStream_t st = begin_launch(stream);
  const bool wf32 = w_dtype == HYC_DTYPE_F32;
  const int64_t P = hyc_rmsnorm_bwd_partials(M, H);
  if (M > 0) {
    if (!dy || !stored || !w || !rstd || !dx || !dw_partials) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null buffer");
    if (d->mode == HYC_MODE_CHANNEL && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null vals/scales");
    if (!aligned16(dy) || !aligned16(dx) || !aligned16(w) || !aligned16(dw_partials) || !aligned8(stored) ||
        (d->mode == HYC_MODE_DENSE && !aligned16(stored)))
      return fail(HYC_EINVAL, "hyc_rmsnorm_bwd: dy, dx, w, dw_partials must be 16-byte aligned, stored 8-byte (16 when dense)");
    const int rpb = (int)bwd_rows_per_block(M);
    const uint16_t* gp = static_cast<const uint16_t*>(dy);
    if (d->mode == HYC_MODE_CHANNEL) {
      HYC_BITS_ITERS_MAXT(d->bits, round_iters(g.iters), g.threads,
        hipLaunchKernelGGL((k_rmsnorm_bwd<B, IT, MT, 0>), dim3((unsigned)P), dim3(g.threads), 0, st, gp,
                           static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),
                           static_cast<const uint16_t*>(scales), w, wf32, rstd, M, H, g.cps, rpb, ca, c2_quirk != 0,
                           static_cast<uint16_t*>(dx), dw_partials));
    } else {
      HYC_BITS_ITERS_MAXT(d->bits, round_iters(g.iters), g.threads,
        hipLaunchKernelGGL((k_rmsnorm_bwd<B, IT, MT, 2>), dim3((unsigned)P), dim3(g.threads), 0, st, gp,
                           static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),
                           static_cast<const uint16_t*>(scales), w, wf32, rstd, M, H, g.cps, rpb, ca, c2_quirk != 0,
                           static_cast<uint16_t*>(dx), dw_partials));
    }
    if ((rc = check_launch("hyc_rmsnorm_bwd"))) return rc;
  }
  hipLaunchKernelGGL(k_colsum, dim3((unsigned)((H + 31) / 32)), dim3(256), 0, st, dw_partials, P, H, dw, wf32);
  return check_launch("hyc_rmsnorm_bwd (dw)");
}

}  // extern "C"
