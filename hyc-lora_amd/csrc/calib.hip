// Calibration kernels of the channel mode: per-channel abs-max over the tokens, selection of the k
// largest channels (ties to the lower index, output ascending) and the per-chunk lookup plan that the
// row kernels read.  They run twice per module lifetime, in front of a compress call, so they are kept to a few
// microseconds: one streaming pass for the abs-max, one single-workgroup launch for the selection.
#include "abi_util.hpp"
#include "wave_scan.hpp"

namespace hyc {

// A workgroup of four waves covers 64 chunks (512 channels, 1 KB of a row per wave instruction) over ABSMAX_ROWS rows:
// wave w takes rows w, w + 4, ..., sixteen loads in flight per thread; the four waves' maxima meet in LDS and leave as
// one atomic per channel and workgroup.  |x| of a bf16 compares as an integer.  (A workgroup that walks whole rows of
// 4096 channels front to back, as the compress kernels do, has too few workgroups at calibration sizes: 12.7 us against
// 4.8 us at 2048 x 4096, 93 against 60 at 32 768 rows.)
constexpr int ABSMAX_ROWS = 128, ABSMAX_BATCH = 16;

__global__ void __launch_bounds__(256)
k_channel_absmax(const uint16_t* __restrict__ x, int64_t M, int64_t H, unsigned int* __restrict__ amax_bits) {
  __shared__ uint32_t part[4][64][9];                       // [wave][lane][channel of the chunk], padded
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t cc = (int64_t)blockIdx.x * 64 + lane;
  const int64_t nch = H / 8;
  const int64_t r0 = (int64_t)blockIdx.y * ABSMAX_ROWS + wave;
  const int64_t left = (M - r0) * H * 2;                    // bytes from this wave's first row to the end of x
  const BufferRsrc rs = make_rsrc(x + r0 * H, left <= 0 ? 0u : (uint32_t)(left < ((int64_t)1 << 31) ? left : ((int64_t)1 << 31) - 1));
  const uint32_t off = cc < nch ? (uint32_t)(16 * cc) : NOWHERE;
  const uint32_t row_b = (uint32_t)(H * 2);
  uint32_t m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int b = 0; b < ABSMAX_ROWS / 4 / ABSMAX_BATCH; ++b) {
    uint4 v[ABSMAX_BATCH];
#pragma unroll
    for (int i = 0; i < ABSMAX_BATCH; ++i) v[i] = load_b128(rs, off + (uint32_t)(4 * (b * ABSMAX_BATCH + i)) * row_b);   // rows past the end read zeros
#pragma unroll
    for (int i = 0; i < ABSMAX_BATCH; ++i) {
      const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = w[j] & 0x7FFFu, hi = (w[j] >> 16) & 0x7FFFu;
        m[2 * j] = lo > m[2 * j] ? lo : m[2 * j];
        m[2 * j + 1] = hi > m[2 * j + 1] ? hi : m[2 * j + 1];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) part[wave][lane][j] = m[j];
  __syncthreads();
  // thread t: channel t and t + 256 of the workgroup's 512 (neighbouring threads, neighbouring addresses)
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int ch = (int)threadIdx.x + 256 * u, l = ch >> 3, j = ch & 7;
    uint32_t best = part[0][l][j];
#pragma unroll
    for (int w = 1; w < 4; ++w) best = part[w][l][j] > best ? part[w][l][j] : best;
    const int64_t c = (int64_t)blockIdx.x * 512 + ch;
    // non-negative floats order as unsigned integers; a channel whose running maximum is not exceeded needs no atomic
    if (c < H && (best << 16) > amax_bits[c]) atomicMax(amax_bits + c, best << 16);
  }
}

// ---- selection: one workgroup of 1024 threads ---------------------------------------------------------------------
// selected(c) <=> #{c' : s[c'] > s[c] or (s[c'] == s[c] and c' < c)} < k.  The k-th largest score T is found by a
// radix select over order-preserving 32-bit keys (four passes of 8 bits, most significant first, two when no key has
// bits in its low half: a histogram of the digit of every key that matches the prefix found so far, then the bin that
// holds rank k); the channels above T are
// selected, and of those equal to T the first `need` by index.  Two prefix sums over the workgroup then give the rank of
// every tie and the position of every selected channel, from which the plan words and the ascending list follow.
constexpr int SEL_THREADS = 1024, SEL_LDS_KEYS = 16384;

__device__ __forceinline__ uint32_t score_key(float s) {
  const uint32_t bits = __float_as_uint(s);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

// adds one to lh[bin] for every lane with `on`; a wave whose active lanes all hit one bin adds once
__device__ __forceinline__ void sel_tally(uint32_t* lh, bool on, uint32_t bin) {
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

// exclusive prefix sum of one value per thread over the workgroup; `total` receives the sum.  scratch: 16 ints.
__device__ __forceinline__ int block_exclusive_scan(int v, int* scratch, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int incl = wave_inclusive_scan(v);
  __syncthreads();                                          // scratch may still be read from an earlier scan
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < SEL_THREADS / 64; ++w) { const int t = scratch[w]; all += t; before += w < wave ? t : 0; }
  *total = all;
  return before + incl - v;
}

__global__ void __launch_bounds__(SEL_THREADS)
k_select(const float* __restrict__ amax, int H, int k, uint32_t* __restrict__ plan, int32_t* __restrict__ idx) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t s_prefix, s_need;
  __shared__ int scratch[SEL_THREADS / 64];
  extern __shared__ uint32_t keys[];                        // the keys, when they fit (else they are read again from memory)
  const int tid = threadIdx.x;
  const bool cached = H <= SEL_LDS_KEYS;
  auto key_at = [&](int i) __attribute__((always_inline)) { return cached ? keys[i] : score_key(amax[i]); };
  uint32_t low = 0;                                         // scores that came from bf16 data have no low half:
  for (int i = tid; i < H; i += SEL_THREADS) {              // the two passes over it are then skipped
    const uint32_t key = score_key(amax[i]);
    if (cached) keys[i] = key;
    low |= key & 0xFFFFu;
  }
  if (tid == 0) { s_prefix = 0; s_need = (uint32_t)k; }
  const int last_shift = __syncthreads_or((int)low) ? 0 : 16;
  uint32_t mask = 0;
  const int trips = (H + SEL_THREADS - 1) / SEL_THREADS;    // the same for every lane: sel_tally votes wave-wide
  for (int shift = 24; shift >= last_shift && k > 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    for (int t = 0; t < trips; ++t) {
      const int i = t * SEL_THREADS + tid;
      const bool in = i < H;
      const uint32_t key = in ? key_at(i) : 0u;
      sel_tally(hist, in && (key & mask) == prefix, (key >> shift) & 255u);
    }
    __syncthreads();
    if (tid < 64) {                                         // one wave: the bin, counted from the top, that holds rank `need`
      // lane l owns bins 255 - 4l .. 252 - 4l, so that a prefix sum over the lanes runs from the largest digit down
      uint32_t c[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = hist[255 - 4 * tid - j];
      const int mine = (int)(c[0] + c[1] + c[2] + c[3]);
      int above = wave_inclusive_scan(mine) - mine;         // keys in larger bins than this lane's
      const int need = (int)s_need;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (need > above && need <= above + (int)c[j]) {    // exactly one (lane, j)
          s_prefix = prefix | ((uint32_t)(255 - 4 * tid - j) << shift);
          s_need = (uint32_t)(need - above);
        }
        above += (int)c[j];
      }
    }
    mask |= 255u << shift;
    __syncthreads();
  }
  // T = s_prefix; need = how many of the channels that equal T are taken (the first by index)
  const uint32_t T = k > 0 ? s_prefix : 0xFFFFFFFFu;
  const int need = k > 0 ? (int)s_need : 0;
  const int nch = H / 8;
  const int cpt = (nch + SEL_THREADS - 1) / SEL_THREADS;    // consecutive chunks per thread (at most 8: H <= 65536)
  const int c0 = tid * cpt, c1 = c0 + cpt < nch ? c0 + cpt : nch;
  uint32_t gt[8], eq[8];
  int n_eq = 0;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    gt[u] = 0; eq[u] = 0;
    const int ch = c0 + u;
    if (u < cpt && ch < c1) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t key = key_at(8 * ch + j);
        gt[u] |= (uint32_t)(key > T) << j;
        eq[u] |= (uint32_t)(key == T && k > 0) << j;
      }
      n_eq += __popc(eq[u]);
    }
  }
  int total;
  int tie_rank = block_exclusive_scan(n_eq, scratch, &total);   // ties before this thread's first chunk
  int n_sel = 0;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    uint32_t take = gt[u];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if ((eq[u] >> j) & 1u) { if (tie_rank < need) take |= 1u << j; ++tie_rank; }
    gt[u] = take;
    n_sel += __popc(take);
  }
  int run = block_exclusive_scan(n_sel, scratch, &total);       // selected channels before this thread's first chunk
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int ch = c0 + u;
    if (u < cpt && ch < c1) {
      plan[ch] = gt[u] | ((uint32_t)run << 16);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if ((gt[u] >> j) & 1u) idx[run++] = 8 * ch + j;
    }
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
  dim3 grid((unsigned)((H / 8 + 63) / 64), (unsigned)tiles);
  hipLaunchKernelGGL(k_channel_absmax, grid, dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(x), M, H, reinterpret_cast<unsigned int*>(amax));
  return check_launch("hyc_channel_absmax");
}

int hyc_select_channels(const float* amax, int64_t H, int32_t k, int32_t* idx, uint32_t* plan, void* stream) {
  if (H <= 0 || H % 8 != 0 || H > 65536) return fail(HYC_EINVAL, "hyc_select_channels: H=%lld", (long long)H);
  if (k < 0 || k > H || k > 65535) return fail(HYC_EINVAL, "hyc_select_channels: k=%d", k);
  if (!amax || !plan || (k > 0 && !idx)) return fail(HYC_EFAULT, "hyc_select_channels: null buffer");
  hipStream_t st = begin_launch(stream);
  const size_t lds = H <= SEL_LDS_KEYS ? (size_t)H * 4 : 0;
  hipLaunchKernelGGL(k_select, dim3(1), dim3(SEL_THREADS), lds, st, amax, (int)H, (int)k, plan, idx);
  return check_launch("hyc_select_channels");
}

}  // extern "C"
