// k-th smallest value of a large array: the calibration quantile of the reference
// (`torch.kthvalue(x[0].flatten().float(), k)`, operators/compress_function.py:319 for activations and :345 for the
// attention probabilities).  Radix select over order-preserving 32-bit keys, 8 bits per pass, most significant digit
// first: a pass histograms the digit of every element whose higher digits equal the prefix found so far; a one-block
// kernel then picks the bin that holds rank k.  Four passes over fp32 input, two over bf16 (whose keys have only
// 16 significant bits); nothing is sorted, nothing returns to the host.
#include "abi_util.hpp"

namespace hyc {

struct KthState {
  uint32_t hist[256];
  uint32_t prefix, mask, k, pad;
};

__device__ __forceinline__ uint32_t order_key(uint32_t bits) {
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
__device__ __forceinline__ uint32_t key_bits(uint32_t key) {
  return (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key;
}

__global__ void k_kth_init(KthState* st, uint32_t k) {
  st->hist[threadIdx.x] = 0;
  if (threadIdx.x == 0) { st->prefix = 0; st->mask = 0; st->k = k; st->pad = 0; }
}

// adds one to lh[bin] for every lane with `on`; a wave whose active lanes all hit one bin adds once
__device__ __forceinline__ void tally(uint32_t* lh, bool on, uint32_t bin) {
  const unsigned long long act = __ballot(on);
  if (act == 0) return;
  const int first = __ffsll((long long)act) - 1;
  const uint32_t fb = __shfl(bin, first);
  const unsigned long long same = __ballot(on && bin == fb);
  if (same == act) {
    if ((int)(threadIdx.x & 63) == first) atomicAdd(&lh[fb], (uint32_t)__popcll(act));
  } else if (on) {
    atomicAdd(&lh[bin], 1u);
  }
}

template <bool BF16>
__global__ void __launch_bounds__(256)
k_kth_hist(const void* __restrict__ xv, int64_t n, KthState* st, int shift) {
  __shared__ uint32_t lh[256];
  lh[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t prefix = st->prefix, mask = st->mask;
  constexpr int PER = BF16 ? 8 : 4;
  const int64_t nvec = n / PER;
  const uint4* xq = static_cast<const uint4*>(xv);
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x;
  // every lane of a wave runs the same number of trips (tally uses wave-wide votes)
  const int64_t trips = (nvec + stride - 1) / stride;
  for (int64_t it = 0; it < trips; ++it) {
    const int64_t i = first + it * stride;
    const bool in = i < nvec;
    uint4 q = make_uint4(0, 0, 0, 0);
    if (in) q = xq[i];
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (BF16) {
        const uint32_t k0 = order_key(w[j] << 16), k1 = order_key(w[j] & 0xFFFF0000u);
        tally(lh, in && (k0 & mask) == prefix, (k0 >> shift) & 255u);
        tally(lh, in && (k1 & mask) == prefix, (k1 >> shift) & 255u);
      } else {
        const uint32_t k0 = order_key(w[j]);
        tally(lh, in && (k0 & mask) == prefix, (k0 >> shift) & 255u);
      }
    }
  }
  if (blockIdx.x == 0) {                               // the tail that does not fill a 16-byte vector
    const int64_t i = nvec * PER + threadIdx.x;
    const bool in = i < n;
    uint32_t key = 0;
    if (in) key = BF16 ? order_key((uint32_t)static_cast<const uint16_t*>(xv)[i] << 16)
                       : order_key(static_cast<const uint32_t*>(xv)[i]);
    tally(lh, in && (key & mask) == prefix, (key >> shift) & 255u);
  }
  __syncthreads();
  const uint32_t c = lh[threadIdx.x];
  if (c) atomicAdd(&st->hist[threadIdx.x], c);
}

// one block of 256: the bin whose cumulative count first reaches k becomes the next digit of the prefix
__global__ void __launch_bounds__(256)
k_kth_pick(KthState* st, int shift, int last, int bf16, float* out) {
  __shared__ uint32_t cum[256];
  const int t = threadIdx.x;
  const uint32_t mine = st->hist[t];
  cum[t] = mine;
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const uint32_t add = t >= d ? cum[t - d] : 0u;
    __syncthreads();
    cum[t] += add;
    __syncthreads();
  }
  const uint32_t k = st->k, incl = cum[t], excl = incl - mine;
  __syncthreads();
  st->hist[t] = 0;
  if (k > excl && k <= incl) {
    const uint32_t prefix = st->prefix | ((uint32_t)t << shift);
    st->prefix = prefix;
    st->mask = st->mask | (255u << shift);
    st->k = k - excl;
    if (last) {
      uint32_t bits = key_bits(prefix);
      if (bf16) bits &= 0xFFFF0000u;
      *out = __uint_as_float(bits);
    }
  }
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int64_t hyc_kth_value_workspace_bytes(void) { return (int64_t)sizeof(KthState); }

int hyc_kth_value(const void* x, int32_t x_dtype, int64_t n, int64_t k, float* out, void* workspace, void* stream) {
  if (x_dtype != HYC_DTYPE_BF16 && x_dtype != HYC_DTYPE_F32)
    return fail(HYC_ENOTSUP, "hyc_kth_value: x_dtype=%d (bf16 or fp32)", x_dtype);
  if (n <= 0 || n >= (int64_t)1 << 31) return fail(HYC_EINVAL, "hyc_kth_value: n=%lld out of range (1..2^31-1)", (long long)n);
  if (k < 1 || k > n) return fail(HYC_EINVAL, "hyc_kth_value: k=%lld must be in 1..n=%lld", (long long)k, (long long)n);
  if (!x || !out || !workspace) return fail(HYC_EFAULT, "hyc_kth_value: null buffer");
  if (!aligned16(x) || !aligned16(workspace)) return fail(HYC_EINVAL, "hyc_kth_value: x and workspace must be 16-byte aligned");
  hipStream_t st = begin_launch(stream);
  KthState* state = static_cast<KthState*>(workspace);
  const bool bf = x_dtype == HYC_DTYPE_BF16;
  const int64_t nvec = n / (bf ? 8 : 4);
  int64_t blocks = (nvec + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(k_kth_init, dim3(1), dim3(256), 0, st, state, (uint32_t)k);
  const int lowest = bf ? 16 : 0;
  for (int shift = 24; shift >= lowest; shift -= 8) {
    if (bf) hipLaunchKernelGGL(k_kth_hist<true>, dim3((unsigned)blocks), dim3(256), 0, st, x, n, state, shift);
    else hipLaunchKernelGGL(k_kth_hist<false>, dim3((unsigned)blocks), dim3(256), 0, st, x, n, state, shift);
    hipLaunchKernelGGL(k_kth_pick, dim3(1), dim3(256), 0, st, state, shift, shift == lowest ? 1 : 0, bf ? 1 : 0, out);
  }
  return check_launch("hyc_kth_value");
}

}  // extern "C"
