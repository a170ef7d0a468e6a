// Backward of the elementwise operators with the decompression fused in:
//   SiLU      dx = s*(1 + x - x*s)*g, s = sigmoid(x)          operators/efficient_silu.py:50-51
//   GELU      tanh-form derivative                            operators/efficient_gelu.py:49-62
//   Hadamard  dx1 = g*x2, dx2 = x1*g                          operators/efficient_hadamard.py:62-66
// Every intermediate is rounded to bf16 exactly where the reference's torch expression rounds it (each
// torch op on bf16 tensors computes in fp32 and rounds once; Python scalars enter as fp32).
#include "abi_util.hpp"
#include "row_kernels.hpp"

namespace hyc {

constexpr int ACT_MUL = 100;   // dx = g * x_hat (one half of the Hadamard backward)

__device__ __forceinline__ float silu_grad(float x, float g) {
  const float s = bfr(1.0f / (1.0f + expf(-x)));
  const float a = bfr(x + 1.0f);
  const float b = bfr(x * s);
  const float c = bfr(a - b);
  const float d = bfr(s * c);
  return bfr(d * g);
}

__device__ __forceinline__ float gelu_tanh_grad(float x, float g) {
  const float gamma = 0.7978845608028654f;   // sqrt(2/pi)
  const float kappa = 0.044715f;
  const float kappa3 = (float)(3 * 0.044715);
  const float x2 = bfr(x * x);
  const float x3 = bfr(x2 * x);
  const float inner = bfr(gamma * bfr(x + bfr(kappa * x3)));
  const float t = bfr(tanhf(inner));
  const float A = bfr(1.0f + t);
  const float B = bfr(1.0f - bfr(t * t));
  const float C = bfr(B * gamma);
  const float E = bfr(1.0f + bfr(kappa3 * x2));
  const float G = bfr(x * bfr(C * E));
  const float I = bfr(0.5f * bfr(A + G));
  return bfr(I * g);
}

template <int ACT>
__device__ __forceinline__ float act_grad(float x, float g) {
  if (ACT == HYC_ACT_SILU) return silu_grad(x, g);
  if (ACT == HYC_ACT_GELU_TANH) return gelu_tanh_grad(x, g);
  return bfr(g * x);
}

// SRC 0 = channel-compressed, 2 = dense bf16
template <int BITS, int SRC, int ACT>
__global__ void __launch_bounds__(1024)
k_act_bwd(const uint16_t* __restrict__ g, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
          const uint16_t* __restrict__ scales, int64_t M, int64_t H, int CPS, int iters, ChanArgs ca,
          uint16_t* __restrict__ dx) {
  constexpr int NSEG = Q<BITS>::NSEG;
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
          if (SRC == 0) decode_chan<BITS>(pk.x, pk.y, i, c, CPS, ca, vals + row * ca.k, scales + row * ca.groups_per_row, xv);
          else unpack8(*reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(stored) + row * H + col), xv);
          unpack8(graw[i], gv);
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = act_grad<ACT>(xv[j], gv[j]);
          *reinterpret_cast<uint4*>(dx + row * H + col) = pack8(o);
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
  const int grid = (int)(M < cap ? M : cap);
  hipStream_t st = begin_launch(stream);
#define HYC_ACT_LAUNCH(B_, S_)                                                                            \
  hipLaunchKernelGGL((k_act_bwd<B_, S_, ACT>), dim3(grid), dim3(geo.threads), 0, st,                      \
                     static_cast<const uint16_t*>(g), static_cast<const uint8_t*>(stored),                \
                     static_cast<const uint16_t*>(vals), static_cast<const uint16_t*>(scales), M, H, geo.cps, \
                     geo.iters, ca, static_cast<uint16_t*>(dx))
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
  int rc = launch_act<ACT_MUL>(g, stored2, vals2, scales2, M, H, d2, dx1, stream, "hyc_hadamard_bwd(dx1)");
  if (rc) return rc;
  return launch_act<ACT_MUL>(g, stored1, vals1, scales1, M, H, d1, dx2, stream, "hyc_hadamard_bwd(dx2)");
}

}  // extern "C"
