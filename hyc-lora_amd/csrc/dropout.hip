// Seeded dropout that keeps nothing for its backward: the mask is regenerated from (seed, element index)
// (reference: operators/efficient_dropout.py:7-53, kernels written with Triton's tl.rand).  tl.rand (triton
// language/random.py, 3.6.0) is the first word of Philox4x32-10 with counter (index, 0, 0, 0) and key
// (seed low word, seed high word), folded to a non-negative int32 (x < 0 -> -x - 1) and multiplied by
// 4.6566127342e-10; an element is kept when that number is > p.
//   forward   out = keep ? bf16(x / (1 - p)) : 0                      (:24-27)
//   backward  out = keep ? g : 0                                      (:49-52; the reference does not divide here)
// One Philox block per element, as in the reference: the kernel is bound by that arithmetic (about 90 integer
// instructions per element), not by memory.
#include "abi_util.hpp"

namespace hyc {

__device__ __forceinline__ uint32_t philox_first_word(uint32_t index, uint32_t k0, uint32_t k1) {
  uint32_t c0 = index, c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t a = c0, b = c2;
    c0 = __umulhi(0xCD9E8D57u, b) ^ c1 ^ k0;
    c2 = __umulhi(0xD2511F53u, a) ^ c3 ^ k1;
    c1 = 0xCD9E8D57u * b;
    c3 = 0xD2511F53u * a;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

__device__ __forceinline__ bool dropout_keep(uint32_t index, uint32_t k0, uint32_t k1, float p) {
  int32_t v = (int32_t)philox_first_word(index, k0, k1);
  v = v < 0 ? -v - 1 : v;
  return (float)v * 4.6566127342e-10f > p;
}

// 8 elements per lane and trip; `scale` = 1/(1-p) applied as a division by (1-p) to match the reference's rounding
template <bool DIVIDE>
__global__ void __launch_bounds__(256)
k_dropout(const uint16_t* __restrict__ x, uint16_t* __restrict__ out, int64_t n, float p, float keep_prob,
          uint32_t k0, uint32_t k1) {
  const int64_t nvec = n / 8;
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < nvec; t += (int64_t)gridDim.x * 256) {
    float v[8];
    unpack8(*reinterpret_cast<const uint4*>(x + 8 * t), v);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool keep = dropout_keep((uint32_t)(8 * t + j), k0, k1, p);
      v[j] = keep ? (DIVIDE ? v[j] / keep_prob : v[j]) : 0.f;
    }
    *reinterpret_cast<uint4*>(out + 8 * t) = pack8(v);
  }
  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(n - nvec * 8)) {       // the tail that does not fill a vector
    const int64_t i = nvec * 8 + threadIdx.x;
    const bool keep = dropout_keep((uint32_t)i, k0, k1, p);
    const float xv = bf_to_f(x[i]);
    out[i] = f_to_bf(keep ? (DIVIDE ? xv / keep_prob : xv) : 0.f);
  }
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_dropout(const void* x, void* out, int64_t n, float p, uint64_t seed, int32_t backward, void* stream) {
  if (n < 0 || n >= ((int64_t)1 << 31)) return fail(HYC_EINVAL, "hyc_dropout: n=%lld out of range (0..2^31-1)", (long long)n);
  if (!(p >= 0.f && p < 1.f)) return fail(HYC_EINVAL, "hyc_dropout: p=%g must be in [0, 1)", (double)p);
  if (n == 0) return HYC_OK;
  if (!x || !out) return fail(HYC_EFAULT, "hyc_dropout: null buffer");
  if (!aligned16(x) || !aligned16(out)) return fail(HYC_EINVAL, "hyc_dropout: x and out must be 16-byte aligned");
  int64_t blocks = (n / 8 + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (blocks < 1) blocks = 1;
  hipStream_t st = begin_launch(stream);
  const uint32_t k0 = (uint32_t)(seed & 0xFFFFFFFFull), k1 = (uint32_t)(seed >> 32);
  const float keep_prob = 1.0f - p;
  if (backward)
    hipLaunchKernelGGL((k_dropout<false>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const uint16_t*>(x),
                       static_cast<uint16_t*>(out), n, p, keep_prob, k0, k1);
  else
    hipLaunchKernelGGL((k_dropout<true>), dim3((unsigned)blocks), dim3(256), 0, st, static_cast<const uint16_t*>(x),
                       static_cast<uint16_t*>(out), n, p, keep_prob, k0, k1);
  return check_launch("hyc_dropout");
}

}  // extern "C"
