// Standalone compress / decompress of a [M, H] bf16 activation, and the element-threshold outliers as CSR.
// One workgroup walks rows (grid-stride); within a row the chunk mapping of row_codec.hpp applies.
#include <stdlib.h>

#include "abi_util.hpp"
#include "row_kernels.hpp"
#include "wave_scan.hpp"

namespace hyc {

// ------------------------------------------------------------------------------------------------
// channel mode
// ------------------------------------------------------------------------------------------------
template <int BITS>
__global__ void __launch_bounds__(1024)
k_compress_chan(const uint16_t* __restrict__ x, int64_t M, int64_t H /* row pitch of x */, int CPS, int iters, int lpg, ChanArgs a,
                uint8_t* __restrict__ stored, uint16_t* __restrict__ vals, uint16_t* __restrict__ scales) {
  constexpr int NSEG = Q<BITS>::NSEG;
  const int64_t SEG = (int64_t)CPS * 8;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* xr = x + row * H;
    uint8_t* sr = stored + row * SEG;
    uint16_t* vr = vals + row * a.k;
    uint16_t* scr = scales + row * a.groups_per_row;
    for (int it = 0; it < iters; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      const bool active = c < CPS;
      uint4 raw[NSEG];
#pragma unroll
      for (int i = 0; i < NSEG; ++i)
        raw[i] = active ? *reinterpret_cast<const uint4*>(xr + i * SEG + 8 * c) : make_uint4(0, 0, 0, 0);
      uint32_t lo, hi;
      encode_chan<BITS>(raw, active, c, CPS, lpg, a, vr, scr, lo, hi);
      if (active) *reinterpret_cast<uint2*>(sr + 8 * c) = make_uint2(lo, hi);
    }
  }
}

template <int BITS>
__global__ void __launch_bounds__(1024)
k_decompress_chan(const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
                  const uint16_t* __restrict__ scales, int64_t M, int64_t H, int CPS, int iters, ChanArgs a,
                  uint16_t* __restrict__ xhat) {
  constexpr int NSEG = Q<BITS>::NSEG;
  const int64_t SEG = (int64_t)CPS * 8;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint8_t* sr = stored + row * SEG;
    const uint16_t* vr = vals + row * a.k;
    const uint16_t* scr = scales + row * a.groups_per_row;
    uint16_t* xr = xhat + row * H;
    for (int it = 0; it < iters; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
        const uint2 w = *reinterpret_cast<const uint2*>(sr + 8 * c);
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          store_stream(xr + i * SEG + 8 * c, decode_chan_pk<BITS>(w.x, w.y, i, c, CPS, a, vr, scr));
        }
      }
    }
  }
}

// Fast paths: every lane owns exactly one chunk per segment (CPS == blockDim.x), the group width is a template
// parameter, plan words are loaded once, pointers advance by a constant and the next row is requested before the
// current one is processed.
template <int BITS, int LPGT, int MAXT, int RULE>
__global__ void __launch_bounds__(MAXT)
k_compress_chan_fast(const uint16_t* __restrict__ x, int64_t M, int64_t H /* row pitch of x */, int CPS, ChanArgs a,
                     uint8_t* __restrict__ stored, uint16_t* __restrict__ vals, uint16_t* __restrict__ scales) {
  constexpr int NSEG = Q<BITS>::NSEG;
  const int c = threadIdx.x;
  if (c >= CPS) return;                                 // tail of the last wave; scale groups never straddle it
  const int64_t SEG = (int64_t)CPS * 8;
  const bool leader = (c & (LPGT - 1)) == 0;
  const int seg_groups = CPS >> a.chunk_to_group_shift;
  uint32_t km[NSEG][4];
  {
    uint32_t plan[NSEG];
#pragma unroll
    for (int i = 0; i < NSEG; ++i) plan[i] = a.plan[i * CPS + c];
    ChunkOutliers<NSEG> co;
    co.init(plan);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km[i]);
  }
  const bool gather = c < a.k;                          // thread c copies outlier channel idx[c] (+ CPS, ...) to vals
  const int idx0 = gather ? a.idx[c] : 0;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint16_t* xrow = x + row * H;
  const uint16_t* xp = xrow + 8 * c;
  uint8_t* sp = stored + row * SEG + 8 * c;
  uint16_t* vp = vals + row * a.k;
  uint16_t* scp = scales + row * a.groups_per_row + (c >> a.chunk_to_group_shift);
  const int64_t xstep = stride * H, sstep = stride * SEG, vstep = stride * a.k, scstep = stride * a.groups_per_row;
  uint4 raw[NSEG];
  uint16_t o = 0;
  if (row < M) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) raw[i] = *reinterpret_cast<const uint4*>(xp + i * SEG);
    if (gather) o = xrow[idx0];
  }
  for (; row < M; row += stride) {
    uint4 nxt[NSEG];
    uint16_t o_n = 0;
    if (row + stride < M) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) nxt[i] = *reinterpret_cast<const uint4*>(xp + xstep + i * SEG);
      if (gather) o_n = xrow[xstep + idx0];
    }
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float v[8];
      unpack8(make_uint4(raw[i].x & km[i][0], raw[i].y & km[i][1], raw[i].z & km[i][2], raw[i].w & km[i][3]), v);
      uint32_t cl, ch;
      const float s = quant_seg<BITS, LPGT, RULE>(v, LPGT, cl, ch, false);
      if (leader) scp[i * seg_groups] = f_to_bf(s);
      if (BITS == 8) { lo = cl; hi = ch; }
      else { lo |= cl << (i * BITS); hi |= ch << (i * BITS); }
    }
    { const u32x2_t t = {lo, hi}; __builtin_nontemporal_store(t, reinterpret_cast<u32x2_t*>(sp)); }   // (read again only in the backward pass)
    if (gather) {
      vp[c] = o;
      for (int t = c + CPS; t < a.k; t += CPS) vp[t] = xrow[a.idx[t]];   // only when k exceeds the workgroup size
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) raw[i] = nxt[i];
    o = o_n;
    xrow += xstep; xp += xstep; sp += sstep; vp += vstep; scp += scstep;
  }
}

template <int BITS, int MAXT>
__global__ void __launch_bounds__(MAXT)
k_decompress_chan_fast(const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
                       const uint16_t* __restrict__ scales, int64_t M, int64_t H, int CPS, ChanArgs a,
                       uint16_t* __restrict__ xhat) {
  constexpr int NSEG = Q<BITS>::NSEG;
  const int c = threadIdx.x;
  if (c >= CPS) return;
  const int64_t SEG = (int64_t)CPS * 8;
  const int seg_groups = CPS >> a.chunk_to_group_shift;
  uint32_t plan[NSEG];
#pragma unroll
  for (int i = 0; i < NSEG; ++i) plan[i] = a.plan[i * CPS + c];
  ChunkOutliers<NSEG> co;
  co.init(plan);
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  const uint8_t* sp = stored + row * SEG + 8 * c;
  const uint16_t* vp = vals + row * a.k;
  const uint16_t* scp = scales + row * a.groups_per_row + (c >> a.chunk_to_group_shift);
  uint16_t* xp = xhat + row * H + 8 * c;
  const int64_t xstep = stride * H, sstep = stride * SEG, vstep = stride * a.k, scstep = stride * a.groups_per_row;
  uint2 pk = make_uint2(0, 0);
  uint32_t sc[NSEG];   // one register each: a packed pair would be assembled right after the load and stall on it
  uint32_t o0[NSEG], o1[NSEG];
  if (row < M) {
    pk = *reinterpret_cast<const uint2*>(sp);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) sc[i] = scp[i * seg_groups];
    co.request(vp, o0, o1);
  }
  for (; row < M; row += stride) {
    uint2 pk_n = make_uint2(0, 0);
    uint32_t sc_n[NSEG], o0_n[NSEG], o1_n[NSEG];
    if (row + stride < M) {
      pk_n = *reinterpret_cast<const uint2*>(sp + sstep);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) sc_n[i] = scp[scstep + i * seg_groups];
      co.request(vp + vstep, o0_n, o1_n);
    }
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      const float sf = bf_to_f((uint16_t)sc[i]);
      uint4 r = co.splice(i, dequant8<BITS>(pk.x, pk.y, i, sf), o0[i], o1[i], sf);
      if (co.more_pairs) r = splice_more(r, co.more_pairs, a.plan[i * CPS + c], vp, true, sf);
      store_stream(xp + i * SEG, r);
    }
    pk = pk_n;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) { sc[i] = sc_n[i]; o0[i] = o0_n[i]; o1[i] = o1_n[i]; }
    xp += xstep; sp += sstep; vp += vstep; scp += scstep;
  }
}

// ------------------------------------------------------------------------------------------------
// threshold mode
// ------------------------------------------------------------------------------------------------
template <int BITS, bool PERCHAN>
__global__ void __launch_bounds__(1024)
k_compress_thr(const uint16_t* __restrict__ x, int64_t M, int64_t H, int CPS, int iters, ThrArgs a,
               uint8_t* __restrict__ stored, int32_t* __restrict__ row_counts) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ float red[16];
  const int64_t SEG = (int64_t)CPS * 8;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* xr = x + row * H;
    uint8_t* sr = stored + row * SEG;
    const int64_t s_pos = row % a.S;
    int hot = 0;
    for (int it = 0; it < iters; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
        uint4 raw[NSEG];
#pragma unroll
        for (int i = 0; i < NSEG; ++i) raw[i] = *reinterpret_cast<const uint4*>(xr + i * SEG + 8 * c);
        uint32_t lo, hi;
        hot += encode_thr<BITS, PERCHAN>(raw, c, CPS, H, s_pos, a, lo, hi);
        *reinterpret_cast<uint2*>(sr + 8 * c) = make_uint2(lo, hi);
      }
    }
    if (row_counts) {                                   // uniform branch
      const float total = block_sum((float)hot, red);   // exact: counts stay far below 2^24
      if (threadIdx.x == 0) row_counts[row] = (int32_t)total;
    }
  }
}

// base at one column (for the outlier fix-up)
__device__ __forceinline__ float base1(const ThrArgs& a, int64_t s_pos, int64_t col, int64_t H) {
  float b = 0.f;
  for (int r = 0; r < a.rank; ++r)
    b = __builtin_fmaf(bf_to_f(a.L[s_pos * a.rank + r]), bf_to_f(a.R[(int64_t)r * H + col]), b);
  return bfr(b);
}

template <int BITS, bool PERCHAN>
__global__ void __launch_bounds__(1024)
k_decompress_thr(const uint8_t* __restrict__ stored, int64_t M, int64_t H, int CPS, int iters, ThrArgs a,
                 uint16_t* __restrict__ xhat) {
  constexpr int NSEG = Q<BITS>::NSEG;
  extern __shared__ __align__(16) uint16_t rowbuf[];     // [H] bf16
  const int64_t SEG = (int64_t)CPS * 8;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint8_t* sr = stored + row * SEG;
    const int64_t s_pos = row % a.S;
    for (int it = 0; it < iters; ++it) {
      const int c = it * blockDim.x + threadIdx.x;
      if (c < CPS) {
        const uint2 w = *reinterpret_cast<const uint2*>(sr + 8 * c);
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          float v[8], b[8];
          decode_thr<BITS, PERCHAN>(w.x, w.y, i, c, CPS, H, s_pos, a, v, b);
          *reinterpret_cast<uint4*>(rowbuf + i * SEG + 8 * c) = pack8(v);
        }
      }
    }
    __syncthreads();
    // the row's outliers: x_hat = bf16(bf16(base + outlier) + dequant)
    const int e0 = a.row_ptr[row], e1 = a.row_ptr[row + 1];
    for (int e = e0 + threadIdx.x; e < e1; e += blockDim.x) {
      const int col = a.cols[e];
      const float o = bf_to_f(a.vals[e]);
      const int i = col / (int)SEG, j = col - i * (int)SEG;
      const int byte = sr[j];
      float q;
      if (BITS == 8) q = (float)(int)(int8_t)byte;
      else q = (float)((int)((byte >> (i * BITS)) & Q<BITS>::CODE_MASK) - Q<BITS>::OFF);
      const float s = bf_to_f(a.scale[s_pos * a.sst + (int64_t)col * a.ssc]);
      const float b = a.rank > 0 ? base1(a, s_pos, col, H) : 0.f;
      rowbuf[col] = f_to_bf(bfr(b + o) + bfr(q * s));
    }
    __syncthreads();
    uint16_t* xr = xhat + row * H;
    for (int cc = threadIdx.x; cc < H / 8; cc += blockDim.x)
      *reinterpret_cast<uint4*>(xr + 8 * cc) = *reinterpret_cast<const uint4*>(rowbuf + 8 * cc);
    __syncthreads();
  }
}

// ---- outliers as CSR ------------------------------------------------------------------------------
// 8-bit mask of the elements of chunk cc (plain column order) that exceed the threshold
// (`raw` = the chunk as loaded)
__device__ __forceinline__ uint32_t hot_mask8_of(const uint4& raw, int64_t cc, int64_t H, int64_t s_pos,
                                                 const ThrArgs& a, float (&v)[8]) {
  unpack8(raw, v);
  if (a.rank > 0) {
    float b[8];
    base8(a, s_pos, 8 * cc, H, b);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = bfr(v[j] - b[j]);
  }
  uint32_t m = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) m |= (__builtin_fabsf(v[j]) > a.thr) ? (1u << j) : 0u;
  return m;
}
__device__ __forceinline__ uint32_t hot_mask8(const uint16_t* xr, int64_t cc, int64_t H, int64_t s_pos,
                                              const ThrArgs& a, uint4& raw, float (&v)[8]) {
  raw = *reinterpret_cast<const uint4*>(xr + 8 * cc);
  return hot_mask8_of(raw, cc, H, s_pos, a, v);
}

// one wave per row, 4 rows per workgroup
__global__ void __launch_bounds__(256)
k_outlier_count(const uint16_t* __restrict__ x, int64_t M, int64_t H, ThrArgs a, int32_t* __restrict__ counts) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const uint16_t* xr = x + row * H;
  const int64_t s_pos = row % a.S;
  const int64_t nch = H / 8;
  int cnt = 0;
  for (int64_t c0 = 0; c0 < nch; c0 += 64) {
    const int64_t cc = c0 + lane;
    if (cc < nch) {
      uint4 raw; float v[8];
      cnt += __popc(hot_mask8(xr, cc, H, s_pos, a, raw, v));
    }
  }
  const float total = wave_sum((float)cnt);
  if (lane == 0) counts[row] = (int32_t)total;
}

__global__ void __launch_bounds__(256)
k_outlier_fill(const uint16_t* __restrict__ x, int64_t M, int64_t H, ThrArgs a, const int32_t* __restrict__ row_ptr,
               int32_t* __restrict__ cols, uint16_t* __restrict__ vals) {
  __shared__ uint32_t stage_all[4][STAGE_CAP];
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;                                  // whole waves leave together
  uint32_t* stage = stage_all[threadIdx.x >> 6];
  const uint16_t* xr = x + row * H;
  const int64_t s_pos = row % a.S;
  const int64_t nch = H / 8;
  const int64_t base = row_ptr[row];
  const int limit = (int)(row_ptr[row + 1] - base);        // the row's room in cols / vals
  int32_t* cols_row = cols + base;
  uint16_t* vals_row = vals + base;
  int running = 0;
  uint4 next = lane < nch ? *reinterpret_cast<const uint4*>(xr + 8 * lane) : make_uint4(0, 0, 0, 0);
  for (int64_t c0 = 0; c0 < nch; c0 += 64) {
    const int64_t cc = c0 + lane;
    const uint4 raw = next;
    if (cc + 64 < nch) next = *reinterpret_cast<const uint4*>(xr + 8 * (cc + 64));   // the next chunk is on its way
    float v[8];
    uint32_t m = 0;
    if (cc < nch) m = hot_mask8_of(raw, cc, H, s_pos, a, v);
    const int cnt = __popc(m);
    const int incl = wave_inclusive_scan(cnt);           // prefix sum over the wave
    int pos = running + incl - cnt;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((m >> j) & 1u) {
        stage_entry(stage, pos, limit, (int)(8 * cc + j), f_to_bf(v[j]), cols_row, vals_row);   // the value after the base was removed
        ++pos;
      }
    }
    running += __builtin_amdgcn_readlane(incl, 63);
  }
  stage_flush(stage, running, limit, cols_row, vals_row);
}

// ---- launch helpers -------------------------------------------------------------------------------
static inline int row_grid(int64_t M, int threads) {
  // enough workgroups to keep 256 CUs busy with several rows in flight each
  const int per_cu = threads >= 512 ? 3 : 8;
  const int64_t cap = (int64_t)256 * per_cu;
  return (int)(M < cap ? M : cap);
}

// Long inputs: one workgroup per two rows.  The row loops take one row per iteration with the next one requested
// ahead; short loops that the dispatcher balances beat both the default grid and a grid of exactly the resident
// workgroups (65 536 x 4096 INT4: compress 141 -> 121 us, decompress 102 -> 96 us; 16 384 x 11008: 93 -> 83, 71 -> 66;
// threshold scheme, 16 384 x 4096: 36.5 -> 30.7 and 47.0 -> 38.7 us).
static int long_input_grid(int64_t M, int dflt) {
  const int64_t g = M / 2;
  return g > dflt ? (int)g : dflt;
}

#define HYC_DISPATCH_BITS(BITS_, ...)            \
  switch (BITS_) {                               \
    case 1: { constexpr int B = 1; __VA_ARGS__; } break; \
    case 2: { constexpr int B = 2; __VA_ARGS__; } break; \
    case 4: { constexpr int B = 4; __VA_ARGS__; } break; \
    default: { constexpr int B = 8; __VA_ARGS__; } break; \
  }
}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_compress(const void* x, int64_t M, int64_t H, const hyc_desc* d, void* stored, void* vals, void* scales,
                 int32_t* row_counts, void* stream) {
  return hyc_compress_rows(x, H, M, H, d, stored, vals, scales, row_counts, stream);
}

int hyc_compress_rows(const void* x, int64_t ldx, int64_t M, int64_t H, const hyc_desc* d, void* stored, void* vals,
                      void* scales, int32_t* row_counts, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_compress: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_compress: M=%lld", (long long)M);
  if (ldx < H || ldx % 8 != 0 || (d->mode != HYC_MODE_CHANNEL && ldx != H))
    return fail(HYC_EINVAL, "hyc_compress: row pitch %lld (at least H=%lld, a multiple of 8; equal to H outside the channel scheme)",
                (long long)ldx, (long long)H);
  RowGeom g;
  int rc = row_geom(H, d->bits, &g);
  if (rc) return rc;
  hipStream_t st = begin_launch(stream);
  if (d->mode == HYC_MODE_CHANNEL) {
    ChanArgs a; int lpg;
    if ((rc = make_chan_args(d, g, &a, &lpg))) return rc;
    if (M == 0) return HYC_OK;
    if (!x || !stored || !scales || (d->k > 0 && !vals)) return fail(HYC_EFAULT, "hyc_compress: null buffer");
    if (!aligned16(x) || !aligned8(stored)) return fail(HYC_EINVAL, "hyc_compress: x must be 16-byte and stored 8-byte aligned");
    const int grid = row_grid(M, g.threads);
    if (g.iters == 1 && (lpg == 8 || lpg == 16) && d->bits != 1) {
#define HYC_CF_R(B_, L_, R_)                                                                                       \
  do {                                                                                                             \
    if (g.threads <= 256)                                                                                          \
      hipLaunchKernelGGL((k_compress_chan_fast<B_, L_, 256, R_>),                                                  \
                         dim3(long_input_grid(M, grid)), dim3(g.threads), 0, st, \
                         static_cast<const uint16_t*>(x), M, ldx, g.cps, a, static_cast<uint8_t*>(stored),               \
                         static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales));                            \
    else                                                                                                           \
      hipLaunchKernelGGL((k_compress_chan_fast<B_, L_, 1024, R_>),                                                 \
                         dim3(long_input_grid(M, grid)), dim3(g.threads), 0, st, \
                         static_cast<const uint16_t*>(x), M, ldx, g.cps, a, static_cast<uint8_t*>(stored),               \
                         static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales));                            \
  } while (0)
#define HYC_CF(B_, L_)                                           \
  do {                                                           \
    if (a.absmax) HYC_CF_R(B_, L_, SCALE_ABSMAX);                \
    else HYC_CF_R(B_, L_, SCALE_RANGE);                          \
  } while (0)
      switch (d->bits * 100 + lpg) {
        case 208: HYC_CF(2, 8); break;
        case 216: HYC_CF(2, 16); break;
        case 408: HYC_CF(4, 8); break;
        case 416: HYC_CF(4, 16); break;
        case 808: HYC_CF(8, 8); break;
        default: HYC_CF(8, 16); break;
      }
#undef HYC_CF_R
#undef HYC_CF
      return check_launch("hyc_compress");
    }
    HYC_DISPATCH_BITS(d->bits,
      hipLaunchKernelGGL((k_compress_chan<B>), dim3(grid), dim3(g.threads), 0, st,
                         static_cast<const uint16_t*>(x), M, ldx, g.cps, g.iters, lpg, a, static_cast<uint8_t*>(stored),
                         static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales)));
    return check_launch("hyc_compress");
  }
  if (d->mode == HYC_MODE_THRESHOLD) {
    ThrArgs a; bool perchan;
    if ((rc = make_thr_args(d, g, &a, &perchan))) return rc;
    if (M == 0) return HYC_OK;
    if (!x || !stored) return fail(HYC_EFAULT, "hyc_compress: null buffer");
    if (!aligned16(x) || !aligned8(stored)) return fail(HYC_EINVAL, "hyc_compress: x must be 16-byte and stored 8-byte aligned");
    const int grid = long_input_grid(M, row_grid(M, g.threads));
    HYC_DISPATCH_BITS(d->bits,
      if (perchan) hipLaunchKernelGGL((k_compress_thr<B, true>), dim3(grid), dim3(g.threads), 0, st,
                                      static_cast<const uint16_t*>(x), M, H, g.cps, g.iters, a,
                                      static_cast<uint8_t*>(stored), row_counts);
      else hipLaunchKernelGGL((k_compress_thr<B, false>), dim3(grid), dim3(g.threads), 0, st,
                              static_cast<const uint16_t*>(x), M, H, g.cps, g.iters, a,
                              static_cast<uint8_t*>(stored), row_counts));
    return check_launch("hyc_compress");
  }
  return fail(HYC_EINVAL, "hyc_compress: mode=%d", d->mode);
}

int hyc_decompress(const void* stored, const void* vals, const void* scales, int64_t M, int64_t H, const hyc_desc* d,
                   void* xhat, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_decompress: null descriptor");
  if (M < 0) return fail(HYC_EINVAL, "hyc_decompress: M=%lld", (long long)M);
  RowGeom g;
  int rc = row_geom(H, d->bits, &g);
  if (rc) return rc;
  hipStream_t st = begin_launch(stream);
  if (d->mode == HYC_MODE_CHANNEL) {
    ChanArgs a; int lpg;
    if ((rc = make_chan_args(d, g, &a, &lpg))) return rc;
    if (M == 0) return HYC_OK;
    if (!stored || !xhat || !scales || (d->k > 0 && !vals)) return fail(HYC_EFAULT, "hyc_decompress: null buffer");
    if (!aligned16(xhat) || !aligned8(stored)) return fail(HYC_EINVAL, "hyc_decompress: xhat must be 16-byte and stored 8-byte aligned");
    const int grid = row_grid(M, g.threads);
    if (g.iters == 1 && d->bits != 1) {
#define HYC_DF(B_)                                                                                                 \
  do {                                                                                                             \
    if (g.threads <= 256)                                                                                          \
      hipLaunchKernelGGL((k_decompress_chan_fast<B_, 256>),                                                        \
                         dim3(long_input_grid(M, grid)), dim3(g.threads), 0, st, \
                         static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                  \
                         static_cast<const uint16_t*>(scales), M, H, g.cps, a, static_cast<uint16_t*>(xhat));         \
    else                                                                                                           \
      hipLaunchKernelGGL((k_decompress_chan_fast<B_, 1024>),                                                       \
                         dim3(long_input_grid(M, grid)), dim3(g.threads), 0, st, \
                         static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                  \
                         static_cast<const uint16_t*>(scales), M, H, g.cps, a, static_cast<uint16_t*>(xhat));         \
  } while (0)
      if (d->bits == 2) HYC_DF(2);
      else if (d->bits == 4) HYC_DF(4);
      else HYC_DF(8);
#undef HYC_DF
      return check_launch("hyc_decompress");
    }
    HYC_DISPATCH_BITS(d->bits,
      hipLaunchKernelGGL((k_decompress_chan<B>), dim3(grid), dim3(g.threads), 0, st,
                         static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),
                         static_cast<const uint16_t*>(scales), M, H, g.cps, g.iters, a, static_cast<uint16_t*>(xhat)));
    return check_launch("hyc_decompress");
  }
  if (d->mode == HYC_MODE_THRESHOLD) {
    ThrArgs a; bool perchan;
    if ((rc = make_thr_args(d, g, &a, &perchan))) return rc;
    if (M == 0) return HYC_OK;
    if (!stored || !xhat) return fail(HYC_EFAULT, "hyc_decompress: null buffer");
    if (!a.row_ptr) return fail(HYC_EFAULT, "hyc_decompress: threshold mode needs csr_row_ptr");
    if (!aligned16(xhat) || !aligned8(stored)) return fail(HYC_EINVAL, "hyc_decompress: xhat must be 16-byte and stored 8-byte aligned");
    const int grid = long_input_grid(M, row_grid(M, g.threads));
    const size_t lds = (size_t)H * 2;
    HYC_DISPATCH_BITS(d->bits,
      if (perchan) hipLaunchKernelGGL((k_decompress_thr<B, true>), dim3(grid), dim3(g.threads), lds, st,
                                      static_cast<const uint8_t*>(stored), M, H, g.cps, g.iters, a,
                                      static_cast<uint16_t*>(xhat));
      else hipLaunchKernelGGL((k_decompress_thr<B, false>), dim3(grid), dim3(g.threads), lds, st,
                              static_cast<const uint8_t*>(stored), M, H, g.cps, g.iters, a,
                              static_cast<uint16_t*>(xhat)));
    return check_launch("hyc_decompress");
  }
  return fail(HYC_EINVAL, "hyc_decompress: mode=%d", d->mode);
}

static int outlier_args(const char* who, const void* x, int64_t M, int64_t H, const hyc_desc* d, ThrArgs* a) {
  if (!d) return fail(HYC_EFAULT, "%s: null descriptor", who);
  if (d->mode != HYC_MODE_THRESHOLD) return fail(HYC_EINVAL, "%s: threshold mode only", who);
  if (M < 0 || H <= 0 || H % 8 != 0 || H > 65536) return fail(HYC_EINVAL, "%s: M=%lld H=%lld (H must be a multiple of 8)", who, (long long)M, (long long)H);
  RowGeom g; g.H = H;
  // the scale is not read by these kernels; satisfy the checker with a placeholder when absent
  hyc_desc tmp = *d;
  if (!tmp.scale) { tmp.scale = x; tmp.scale_stride_channel = 0; tmp.scale_stride_token = 0; }
  bool perchan;
  return make_thr_args(&tmp, g, a, &perchan);
}

int hyc_ref_outlier_count(const void* x, int64_t M, int64_t H, const hyc_desc* d, int32_t* counts, void* stream) {
  ThrArgs a;
  int rc = outlier_args("hyc_ref_outlier_count", x, M, H, d, &a);
  if (rc) return rc;
  if (M == 0) return HYC_OK;
  if (!x || !counts) return fail(HYC_EFAULT, "hyc_ref_outlier_count: null buffer");
  if (!aligned16(x)) return fail(HYC_EINVAL, "hyc_ref_outlier_count: x must be 16-byte aligned");
  hipLaunchKernelGGL(k_outlier_count, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(x), M, H, a, counts);
  return check_launch("hyc_ref_outlier_count");
}

int hyc_ref_outlier_fill(const void* x, int64_t M, int64_t H, const hyc_desc* d, const int32_t* row_ptr, int32_t* cols,
                         void* vals, void* stream) {
  ThrArgs a;
  int rc = outlier_args("hyc_ref_outlier_fill", x, M, H, d, &a);
  if (rc) return rc;
  if (M == 0) return HYC_OK;
  if (!x || !row_ptr) return fail(HYC_EFAULT, "hyc_ref_outlier_fill: null buffer");
  if (!aligned16(x)) return fail(HYC_EINVAL, "hyc_ref_outlier_fill: x must be 16-byte aligned");
  hipLaunchKernelGGL(k_outlier_fill, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, begin_launch(stream),
                     static_cast<const uint16_t*>(x), M, H, a, row_ptr, cols, static_cast<uint16_t*>(vals));
  return check_launch("hyc_ref_outlier_fill");
}

}  // extern "C"
