// NF4 block-64 storage of the frozen base weights (call sites in the reference: bitsandbytes_fix/_function.py:509
// and :540, `F.dequantize_4bit(B, quant_state)` before each matmul; the quantiser itself lives in bitsandbytes,
// which the reference does not vendor).  Published format: blocks of 64 consecutive weights share one fp32
// abs-max; each weight is stored as the index of the nearest of 16 fixed levels of w / absmax; two indices per
// byte, the first weight of a pair in the high nibble.  Both kernels are pure streaming work.
#include "abi_util.hpp"

namespace hyc {

// the 16 NormalFloat4 levels
__device__ __constant__ float kNF4[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f, -0.28444138169288635f,
    -0.18477343022823334f, -0.09105003625154495f, 0.0f, 0.07958029955625534f, 0.16093020141124725f,
    0.24611230194568634f, 0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f,
    1.0f};

// index of the nearest level: the number of midpoints between neighbouring levels that lie strictly below v
__device__ __forceinline__ uint32_t nf4_code(float v, const float* mid) {
  uint32_t c = 0;
#pragma unroll
  for (int i = 0; i < 15; ++i) c += v > mid[i] ? 1u : 0u;
  return c;
}

// One lane holds 8 consecutive weights, 8 lanes one block of 64.
__global__ void __launch_bounds__(256)
k_nf4_quantize(const uint16_t* __restrict__ w, int64_t nblocks, uint8_t* __restrict__ packed,
               float* __restrict__ absmax) {
  float mid[15];
#pragma unroll
  for (int i = 0; i < 15; ++i) mid[i] = 0.5f * (kNF4[i] + kNF4[i + 1]);
  const int64_t lanes = nblocks * 8;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < lanes; t += (int64_t)gridDim.x * 256) {
    float v[8];
    unpack8(*reinterpret_cast<const uint4*>(w + 8 * t), v);
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(v[j]));
    m = fmaxf(m, __shfl_xor(m, 1));
    m = fmaxf(m, __shfl_xor(m, 2));
    m = fmaxf(m, __shfl_xor(m, 4));
    const float inv = m > 0.f ? 1.0f / m : 0.f;
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      const uint32_t hi = nf4_code(v[j] * inv, mid), lo = nf4_code(v[j + 1] * inv, mid);
      word |= ((hi << 4) | lo) << (4 * j);
    }
    *reinterpret_cast<uint32_t*>(packed + 4 * t) = word;
    if ((t & 7) == 0) absmax[t >> 3] = m;
  }
}

// One lane expands 4 bytes (8 weights) into one 16-byte store, so that a wave reads 256 and writes 1024 contiguous
// bytes per step; four independent steps per trip keep enough loads in flight.
__global__ void __launch_bounds__(256)
k_nf4_dequantize(const uint8_t* __restrict__ packed, const float* __restrict__ absmax, int64_t nwords,
                 uint16_t* __restrict__ out) {
  __shared__ float lut[16];
  if (threadIdx.x < 16) lut[threadIdx.x] = kNF4[threadIdx.x];
  __syncthreads();
  const uint32_t* words = reinterpret_cast<const uint32_t*>(packed);
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < nwords; t += 4 * step) {
    uint32_t w[4];
    float s[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = t + u * step;
      const bool on = i < nwords;
      w[u] = on ? words[i] : 0u;
      s[u] = on ? absmax[i >> 3] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = t + u * step;
      if (i >= nwords) break;
      float v[8];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (w[u] >> (8 * b)) & 0xFFu;
        v[2 * b] = lut[byte >> 4] * s[u];
        v[2 * b + 1] = lut[byte & 15u] * s[u];
      }
      *reinterpret_cast<uint4*>(out + 8 * i) = pack8(v);
    }
  }
}

static int nf4_args(const char* who, int64_t n, const void* a, const void* b, const void* c) {
  if (n < 0 || n % 64 != 0) return fail(HYC_EINVAL, "%s: n=%lld must be a non-negative multiple of 64", who, (long long)n);
  if (n == 0) return HYC_OK;
  if (!a || !b || !c) return fail(HYC_EFAULT, "%s: null buffer", who);
  return HYC_OK;
}

static unsigned stream_grid(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  return (unsigned)blocks;
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_nf4_quantize(const void* w, int64_t n, void* packed, float* absmax, void* stream) {
  int rc = nf4_args("hyc_nf4_quantize", n, w, packed, absmax);
  if (rc || n == 0) return rc;
  if (!aligned16(w) || (reinterpret_cast<uintptr_t>(packed) & 3u))
    return fail(HYC_EINVAL, "hyc_nf4_quantize: w must be 16-byte and packed 4-byte aligned");
  const int64_t nblocks = n / 64;
  hipLaunchKernelGGL(k_nf4_quantize, dim3(stream_grid(nblocks * 8)), dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(w), nblocks, static_cast<uint8_t*>(packed), absmax);
  return check_launch("hyc_nf4_quantize");
}

int hyc_nf4_dequantize(const void* packed, const float* absmax, int64_t n, void* out, void* stream) {
  int rc = nf4_args("hyc_nf4_dequantize", n, packed, absmax, out);
  if (rc || n == 0) return rc;
  if (!aligned16(packed) || !aligned16(out))
    return fail(HYC_EINVAL, "hyc_nf4_dequantize: packed and out must be 16-byte aligned");
  const int64_t nblocks = n / 64;
  hipLaunchKernelGGL(k_nf4_dequantize, dim3(stream_grid(nblocks * 2)), dim3(256), 0, begin_launch(stream),
                     static_cast<const uint8_t*>(packed), absmax, nblocks * 8, static_cast<uint16_t*>(out));
  return check_launch("hyc_nf4_dequantize");
}

}  // extern "C"
