// Calibration kernels of the channel mode: per-channel abs-max over the tokens, selection of the k
// largest channels (ties to the lower index, output ascending) and the per-chunk lookup plan that the
// row kernels read.  These run a couple of times per module lifetime; they are written for clarity.
#include "abi_util.hpp"

namespace hyc {

constexpr int ABSMAX_ROWS = 32;

// grid (ceil(H/8/256), ceil(M/ABSMAX_ROWS)); thread = one 8-channel chunk over a tile of rows
__global__ void __launch_bounds__(256)
k_channel_absmax(const uint16_t* __restrict__ x, int64_t M, int64_t H, unsigned int* __restrict__ amax_bits) {
  const int64_t cc = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (cc >= H / 8) return;
  const int64_t r0 = (int64_t)blockIdx.y * ABSMAX_ROWS;
  const int64_t r1 = r0 + ABSMAX_ROWS < M ? r0 + ABSMAX_ROWS : M;
  uint32_t m[8] = {0, 0, 0, 0, 0, 0, 0, 0};                 // |x| as bf16 bit patterns: monotone as integers
  for (int64_t r = r0; r < r1; ++r) {
    const uint4 v = *reinterpret_cast<const uint4*>(x + r * H + 8 * cc);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = w[j] & 0x7FFFu, hi = (w[j] >> 16) & 0x7FFFu;
      m[2 * j] = lo > m[2 * j] ? lo : m[2 * j];
      m[2 * j + 1] = hi > m[2 * j + 1] ? hi : m[2 * j + 1];
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) atomicMax(amax_bits + 8 * cc + j, m[j] << 16);   // non-negative floats order as uints
}

// selected(c) <=> #{c' : s[c'] > s[c] or (s[c'] == s[c] and c' < c)} < k ; mask byte per chunk into plan's low byte.
// A workgroup ranks 32 channels; its 8 sub-groups of 32 threads each count over one eighth of every tile of scores,
// and the eight partial ranks of a channel are added through LDS.
constexpr int RANK_CH = 32, RANK_SUB = 8, RANK_TILE = 4096;
__global__ void __launch_bounds__(256)
k_select_rank(const float* __restrict__ amax, int H, int k, uint32_t* __restrict__ plan) {
  __shared__ float tile[RANK_TILE];
  __shared__ int part[RANK_SUB][RANK_CH];
  const int ch = threadIdx.x & (RANK_CH - 1), sub = threadIdx.x / RANK_CH;
  const int c = blockIdx.x * RANK_CH + ch;
  const float my = c < H ? amax[c] : 0.f;
  int rank = 0;
  constexpr int SPAN = RANK_TILE / RANK_SUB;
  for (int base = 0; base < H; base += RANK_TILE) {
#pragma unroll
    for (int u = 0; u < RANK_TILE / 256; ++u) {
      const int i = base + u * 256 + threadIdx.x;
      tile[u * 256 + threadIdx.x] = i < H ? amax[i] : -1.f;
    }
    __syncthreads();
    const int first = sub * SPAN;
#pragma unroll 8
    for (int i = 0; i < SPAN; ++i) {
      const float s = tile[first + i];
      rank += (s > my || (s == my && base + first + i < c)) ? 1 : 0;
    }
    __syncthreads();
  }
  part[sub][ch] = rank;
  __syncthreads();
  if (threadIdx.x < RANK_CH) {
    int total = 0;
#pragma unroll
    for (int u = 0; u < RANK_SUB; ++u) total += part[u][threadIdx.x];
    const bool sel = (c < H) && (total < k);
    const unsigned long long ballot = __ballot(sel);
    const int lane = threadIdx.x & 63;
    if ((lane & 7) == 0 && c < H) plan[c >> 3] = (uint32_t)((ballot >> lane) & 0xFFull);
  }
}

// one workgroup: prefix counts into plan's high half, ascending channel list into idx
__global__ void __launch_bounds__(1024)
k_select_finish(int H, uint32_t* __restrict__ plan, int32_t* __restrict__ idx) {
  __shared__ int cnt[1024];
  const int nch = H / 8;
  const int cpt = (nch + 1023) / 1024;
  const int c0 = threadIdx.x * cpt;
  const int c1 = c0 + cpt < nch ? c0 + cpt : nch;
  int mine = 0;
  for (int ch = c0; ch < c1; ++ch) mine += __popc(plan[ch] & 0xFFu);
  cnt[threadIdx.x] = mine;
  __syncthreads();
  int run = 0;
  for (int t = 0; t < (int)threadIdx.x; ++t) run += cnt[t];
  for (int ch = c0; ch < c1; ++ch) {
    const uint32_t m8 = plan[ch] & 0xFFu;
    plan[ch] = m8 | ((uint32_t)run << 16);
    for (int j = 0; j < 8; ++j)
      if ((m8 >> j) & 1u) idx[run++] = 8 * ch + j;
  }
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_channel_absmax(const void* x, int64_t M, int64_t H, float* amax, void* stream) {
  if (M < 0 || H <= 0 || H % 8 != 0 || H > 65536)
    return fail(HYC_EINVAL, "hyc_channel_absmax: M=%lld H=%lld (H must be a multiple of 8, at most 65536)", (long long)M, (long long)H);
  if (M == 0) return HYC_OK;
  if (!x || !amax) return fail(HYC_EFAULT, "hyc_channel_absmax: null buffer");
  if (!aligned16(x)) return fail(HYC_EINVAL, "hyc_channel_absmax: x must be 16-byte aligned");
  const int64_t tiles = (M + ABSMAX_ROWS - 1) / ABSMAX_ROWS;
  if (tiles > 65535) {
    // walk the matrix in slabs the grid's y dimension can cover
    const int64_t slab = (int64_t)65535 * ABSMAX_ROWS;
    for (int64_t r = 0; r < M; r += slab) {
      const int64_t m = M - r < slab ? M - r : slab;
      int rc = hyc_channel_absmax(static_cast<const uint16_t*>(x) + r * H, m, H, amax, stream);
      if (rc) return rc;
    }
    return HYC_OK;
  }
  dim3 grid((unsigned)((H / 8 + 255) / 256), (unsigned)tiles);
  hipLaunchKernelGGL(k_channel_absmax, grid, dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(x), M, H, reinterpret_cast<unsigned int*>(amax));
  return check_launch("hyc_channel_absmax");
}

int hyc_select_channels(const float* amax, int64_t H, int32_t k, int32_t* idx, uint32_t* plan, void* stream) {
  if (H <= 0 || H % 8 != 0 || H > 65536) return fail(HYC_EINVAL, "hyc_select_channels: H=%lld", (long long)H);
  if (k < 0 || k > H || k > 65535) return fail(HYC_EINVAL, "hyc_select_channels: k=%d", k);
  if (!amax || !plan || (k > 0 && !idx)) return fail(HYC_EFAULT, "hyc_select_channels: null buffer");
  hipStream_t st = begin_launch(stream);
  hipLaunchKernelGGL(k_select_rank, dim3((unsigned)((H + RANK_CH - 1) / RANK_CH)), dim3(256), 0, st, amax, (int)H, (int)k, plan);
  hipLaunchKernelGGL(k_select_finish, dim3(1), dim3(1024), 0, st, (int)H, plan, idx);
  return check_launch("hyc_select_channels");
}

}  // extern "C"
