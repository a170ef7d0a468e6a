// x -/+ L @ R fused into one pass (reference: low_rank_extraction / low_rank_addition,
// operators/fused_compression.py:80-99 and :184-210): the rank-r product is accumulated in fp32, applied to
// the fp32 value of x and rounded to bf16 once.  The reference keeps these two functions but never calls them.
#include "abi_util.hpp"

namespace hyc {

// grid-stride over 8-column chunks of the [B*S, H] matrix; row m uses L[m mod S, :]
__global__ void __launch_bounds__(256)
k_low_rank(const uint16_t* __restrict__ L, const uint16_t* __restrict__ R, const uint16_t* __restrict__ x,
           uint16_t* __restrict__ out, int64_t M, int64_t S, int64_t H, int rank, float sign) {
  const int64_t nch = H / 8, total = M * nch;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    const int64_t m = idx / nch, c = idx - m * nch, s = m % S;
    float v[8], dot[8];
    unpack8(*reinterpret_cast<const uint4*>(x + m * H + 8 * c), v);
#pragma unroll
    for (int j = 0; j < 8; ++j) dot[j] = 0.f;
    for (int r = 0; r < rank; ++r) {
      const float l = bf_to_f(L[s * rank + r]);
      float rv[8];
      unpack8(*reinterpret_cast<const uint4*>(R + (int64_t)r * H + 8 * c), rv);
#pragma unroll
      for (int j = 0; j < 8; ++j) dot[j] = __builtin_fmaf(l, rv[j], dot[j]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = v[j] + sign * dot[j];
    *reinterpret_cast<uint4*>(out + m * H + 8 * c) = pack8(v);
  }
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_low_rank_update(const void* L, const void* R, const void* x, void* out, int64_t M, int64_t S, int64_t H,
                        int32_t rank, int32_t subtract, void* stream) {
  if (M < 0 || S <= 0 || H <= 0 || H % 8 != 0 || rank < 0)
    return fail(HYC_EINVAL, "hyc_low_rank_update: M=%lld S=%lld H=%lld rank=%d (H must be a multiple of 8)",
                (long long)M, (long long)S, (long long)H, rank);
  if (M == 0) return HYC_OK;
  if (!x || !out || (rank > 0 && (!L || !R))) return fail(HYC_EFAULT, "hyc_low_rank_update: null buffer");
  if (!aligned16(x) || !aligned16(out) || (rank > 0 && !aligned16(R)))
    return fail(HYC_EINVAL, "hyc_low_rank_update: x, out and R must be 16-byte aligned");
  const int64_t total = M * (H / 8);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(k_low_rank, dim3((unsigned)blocks), dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(L), static_cast<const uint16_t*>(R), static_cast<const uint16_t*>(x),
                     static_cast<uint16_t*>(out), M, S, H, (int)rank, subtract ? -1.0f : 1.0f);
  return check_launch("hyc_low_rank_update");
}

}  // extern "C"
