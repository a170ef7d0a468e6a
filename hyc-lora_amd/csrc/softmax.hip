// Softmax over the last dimension with the sparsified copy for backward.
//   forward   y = softmax(x) (fp32 math, one rounding to bf16); per-row count of y > threshold
//   fill      the kept probabilities as CSR (cols ascending within a row, values verbatim)
//   backward  dx = (g - sum_j g_j*yh_j) * yh, yh = the kept probabilities, zero elsewhere
//   dense     yh as a dense matrix (what true_decompress_softmax returns)
// Reference: operators/efficient_softmax.py:10-45, operators/compress_function.py:264-275.
#include "abi_util.hpp"
#include "wave_scan.hpp"

namespace hyc {

// one workgroup (256 threads) per row, grid-stride; N a multiple of 8
__global__ void __launch_bounds__(256)
k_softmax_fwd(const uint16_t* __restrict__ x, int64_t rows, int64_t N, float thr, uint16_t* __restrict__ y,
              int32_t* __restrict__ counts) {
  __shared__ float red[32];
  const int64_t nch = N / 8;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const uint16_t* xr = x + row * N;
    // pass 1: row maximum
    float m = -INFINITY;
    for (int64_t c = threadIdx.x; c < nch; c += 256) {
      float v[8];
      unpack8(*reinterpret_cast<const uint4*>(xr + 8 * c), v);
#pragma unroll
      for (int j = 0; j < 8; ++j) m = v[j] > m ? v[j] : m;
    }
    m = group_reduce<64>(m, OpMax());
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    // pass 2: sum of exp(x - m)   (the row is re-read from cache)
    float l = 0.f;
    for (int64_t c = threadIdx.x; c < nch; c += 256) {
      float v[8];
      unpack8(*reinterpret_cast<const uint4*>(xr + 8 * c), v);
#pragma unroll
      for (int j = 0; j < 8; ++j) l += expf(v[j] - m);
    }
    l = block_sum(l, red);
    // pass 3: y and the count of kept entries
    int kept = 0;
    uint16_t* yr = y + row * N;
    for (int64_t c = threadIdx.x; c < nch; c += 256) {
      float v[8];
      unpack8(*reinterpret_cast<const uint4*>(xr + 8 * c), v);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[j] = bfr(expf(v[j] - m) / l);
        kept += (v[j] > thr) ? 1 : 0;
      }
      store_stream(yr + 8 * c, pack8(v));
    }
    if (counts) {
      const float total = block_sum((float)kept, red);
      if (threadIdx.x == 0) counts[row] = (int32_t)total;
    }
  }
}

// Rows of up to 4096 entries: one wave per row, the row stays in registers (CPL chunks of 8 per lane), wave-level
// reductions only (no barrier), exp evaluated once per element, the next row requested before this one is processed.
// CAUSAL: row r belongs to query position r % period and sees columns 0..position only; the rest of the row is
// neither read (x may hold anything there) nor exponentiated, and comes out as exact zeros.
// FULL: the row is exactly 512 CPL entries, every lane owns CPL chunks and nothing is predicated on that.
template <int CPL, bool CAUSAL, bool FULL>
__global__ void __launch_bounds__(256)
k_softmax_fwd_wave(const uint16_t* x, int64_t rows, int64_t N, float thr, uint16_t* y,   // y may be x (in place)
                   int32_t* __restrict__ counts, int64_t period) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int nch = (int)(N / 8);
  const int64_t stride = (int64_t)gridDim.x * 4;
  int64_t row = (int64_t)blockIdx.x * 4 + wave;
  bool on[CPL];
#pragma unroll
  for (int u = 0; u < CPL; ++u) on[u] = FULL || lane + 64 * u < nch;
  // last visible column of the current row (everything when not causal); rows advance by a fixed stride, so the
  // position advances by stride mod period with one conditional subtraction
  const int per = CAUSAL ? (int)period : 1;
  const int step = CAUSAL ? (int)(stride % period) : 0;
  int pos = CAUSAL && row < rows ? (int)(row % period) : 0;
  auto wrap = [&](int p) __attribute__((always_inline)) { return p >= per ? p - per : p; };
  uint4 raw[CPL];
  if (row < rows) {
    const int lc = CAUSAL ? pos : (int)N - 1;
#pragma unroll
    for (int u = 0; u < CPL; ++u)
      raw[u] = on[u] && 8 * (lane + 64 * u) <= lc ? *reinterpret_cast<const uint4*>(x + row * N + 8 * (lane + 64 * u))
                                                  : make_uint4(0, 0, 0, 0);
  }
  for (; row < rows; row += stride) {
    uint4 nxt[CPL];
    const int pos_next = wrap(pos + step);
    if (row + stride < rows) {
      const int lc = CAUSAL ? pos_next : (int)N - 1;
#pragma unroll
      for (int u = 0; u < CPL; ++u)
        nxt[u] = on[u] && 8 * (lane + 64 * u) <= lc
                     ? *reinterpret_cast<const uint4*>(x + (row + stride) * N + 8 * (lane + 64 * u)) : make_uint4(0, 0, 0, 0);
    }
    float v[CPL][8];
    float m = -INFINITY;
    const int lc = CAUSAL ? pos : (int)N - 1;
    pos = pos_next;
    // a 512-column slice of the row (one chunk per lane) that lies wholly beyond the position is skipped by the
    // whole wave: no max, no exp, zeros stored
    bool live[CPL];
#pragma unroll
    for (int u = 0; u < CPL; ++u) live[u] = !CAUSAL || 512 * u <= lc;
#pragma unroll
    for (int u = 0; u < CPL; ++u) {
      if (!live[u]) continue;
      unpack8(raw[u], v[u]);
      if (CAUSAL) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[u][j] = 8 * (lane + 64 * u) + j <= lc ? v[u][j] : -INFINITY;
      }
      if (on[u]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) m = v[u][j] > m ? v[u][j] : m;
      }
    }
    m = group_reduce<64>(m, OpMax());
    float l = 0.f;
#pragma unroll
    for (int u = 0; u < CPL; ++u) {
      if (!live[u]) continue;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // the clamp keeps x*log2(e) finite for mask values near the bottom of the bf16 range (e^-128 is 0 in fp32)
        v[u][j] = on[u] ? exp_fast(fmaxf(v[u][j] - m, -128.f)) : 0.f;
        l += v[u][j];
      }
    }
    l = wave_sum(l);
    const float inv = 1.0f / l;
    int kept = 0;
#pragma unroll
    for (int u = 0; u < CPL; ++u) {
      if (live[u]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          v[u][j] = bfr(v[u][j] * inv);
          kept += (v[u][j] > thr) ? 1 : 0;
        }
        if (on[u]) store_stream(y + row * N + 8 * (lane + 64 * u), pack8(v[u]));
      } else if (on[u]) {
        kept += 0.f > thr ? 8 : 0;
        store_stream(y + row * N + 8 * (lane + 64 * u), make_uint4(0, 0, 0, 0));
      }
    }
    if (counts) {
      const float total = wave_sum((float)kept);
      if (lane == 0) counts[row] = (int32_t)total;
    }
#pragma unroll
    for (int u = 0; u < CPL; ++u) raw[u] = nxt[u];
  }
}

// counts only, for probabilities computed elsewhere; one wave per row
__global__ void __launch_bounds__(256)
k_softmax_count(const uint16_t* __restrict__ y, int64_t rows, int64_t N, float thr, int32_t* __restrict__ counts) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint16_t* yr = y + row * N;
  int kept = 0;
  for (int64_t c = lane; c < N / 8; c += 64) {
    float v[8];
    unpack8(*reinterpret_cast<const uint4*>(yr + 8 * c), v);
#pragma unroll
    for (int j = 0; j < 8; ++j) kept += (v[j] > thr) ? 1 : 0;
  }
  const float total = wave_sum((float)kept);
  if (lane == 0) counts[row] = (int32_t)total;
}

// Row offsets of a CSR structure from the per-row counts, in one workgroup: row_ptr[r] = min(capacity, counts[0] + ... +
// counts[r - 1]) for r = 0 .. rows, and the uncut total.  The kernel is as long as its trips to memory, so a thread
// asks for all it can hold at once: 32 768 counts are one round of eight 16-byte loads per thread (sub-tile j =
// counts 4096 j .. 4096 j + 4095, four neighbouring counts per thread: loads and stores contiguous across the wave).
// The thread sums of every sub-tile are scanned over the wave (DPP), the wave totals of all sub-tiles meet in LDS behind
// one barrier, and a 64-bit carry runs through the sub-tiles and on to the next 32 768 counts (the total may exceed
// what the buffers hold).  VEC: counts and row_ptr are 16-byte aligned.
constexpr int OFFS_THREADS = 1024, OFFS_SUB = 8, OFFS_TILE = OFFS_THREADS * 4;
template <bool VEC>
__global__ void __launch_bounds__(OFFS_THREADS)
k_csr_offsets(const int32_t* __restrict__ counts, int64_t rows, int64_t capacity, int32_t* __restrict__ row_ptr,
              int64_t* __restrict__ total) {
  __shared__ int tot[OFFS_SUB][OFFS_THREADS / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  long long carry = 0;
  for (int64_t base = 0; base < rows; base += (int64_t)OFFS_SUB * OFFS_TILE) {
    int c[OFFS_SUB][4], sum[OFFS_SUB], incl[OFFS_SUB];
#pragma unroll
    for (int j = 0; j < OFFS_SUB; ++j) {
      const int64_t i = base + (int64_t)j * OFFS_TILE + 4 * tid;
      if (VEC && i + 3 < rows) {
        const int4 v = *reinterpret_cast<const int4*>(counts + i);
        c[j][0] = v.x; c[j][1] = v.y; c[j][2] = v.z; c[j][3] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) c[j][e] = i + e < rows ? counts[i + e] : 0;
      }
    }
#pragma unroll
    for (int j = 0; j < OFFS_SUB; ++j) {
      sum[j] = (c[j][0] + c[j][1]) + (c[j][2] + c[j][3]);
      incl[j] = wave_inclusive_scan(sum[j]);
      if (lane == 63) tot[j][wave] = incl[j];
    }
    __syncthreads();
    long long run = carry;                                  // entries before sub-tile j
#pragma unroll
    for (int j = 0; j < OFFS_SUB; ++j) {
      int before = 0, all = 0;
#pragma unroll
      for (int w = 0; w < OFFS_THREADS / 64; ++w) { const int t = tot[j][w]; all += t; before += w < wave ? t : 0; }
      long long at = run + before + incl[j] - sum[j];
      const int64_t i = base + (int64_t)j * OFFS_TILE + 4 * tid;
      int o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) { o[e] = (int32_t)(at < capacity ? at : capacity); at += c[j][e]; }
      if (VEC && i + 3 < rows) {
        *reinterpret_cast<int4*>(row_ptr + i) = make_int4(o[0], o[1], o[2], o[3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) if (i + e < rows) row_ptr[i + e] = o[e];
      }
      run += all;
    }
    carry = run;
    __syncthreads();                                        // tot is written again by the next round
  }
  if (tid == 0) {
    row_ptr[rows] = (int32_t)(carry < capacity ? carry : capacity);
    if (total) *total = carry;
  }
}

// one wave per row: ordered compaction of the kept entries (prefix sum over the lanes, entries staged in LDS and
// stored as contiguous runs)
__global__ void __launch_bounds__(256)
k_softmax_fill(const uint16_t* __restrict__ y, int64_t rows, int64_t N, float thr, const int32_t* __restrict__ row_ptr,
               int32_t* __restrict__ cols, uint16_t* __restrict__ vals) {
  __shared__ uint32_t stage_all[4][STAGE_CAP];
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;                               // whole waves leave together
  uint32_t* stage = stage_all[threadIdx.x >> 6];
  const uint16_t* yr = y + row * N;
  const int64_t nch = N / 8;
  const int64_t base = row_ptr[row];
  const int limit = (int)(row_ptr[row + 1] - base);        // the row's room in cols / vals
  int32_t* cols_row = cols + base;
  uint16_t* vals_row = vals + base;
  int running = 0;
  uint4 next = lane < nch ? *reinterpret_cast<const uint4*>(yr + 8 * lane) : make_uint4(0, 0, 0, 0);
  for (int64_t c0 = 0; c0 < nch; c0 += 64) {
    const int64_t c = c0 + lane;
    const uint4 raw = next;
    if (c + 64 < nch) next = *reinterpret_cast<const uint4*>(yr + 8 * (c + 64));   // the next chunk is on its way
    float v[8];
    uint32_t m = 0;
    if (c < nch) {
      unpack8(raw, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) m |= (v[j] > thr) ? (1u << j) : 0u;
    }
    const int cnt = __popc(m);
    const int incl = wave_inclusive_scan(cnt);
    int pos = running + incl - cnt;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if ((m >> j) & 1u) {
        stage_entry(stage, pos, limit, (int)(8 * c + j), f_to_bf(v[j]), cols_row, vals_row);
        ++pos;
      }
    }
    running += __builtin_amdgcn_readlane(incl, 63);
  }
  stage_flush(stage, running, limit, cols_row, vals_row);
}

// the same for rows of up to 4096 entries with every load of the row issued up front (CPL chunks per lane)
template <int CPL>
__global__ void __launch_bounds__(256)
k_softmax_fill_wave(const uint16_t* __restrict__ y, int64_t rows, int64_t N, float thr, const int32_t* __restrict__ row_ptr,
                    int32_t* __restrict__ cols, uint16_t* __restrict__ vals) {
  __shared__ uint32_t stage_all[4][STAGE_CAP];
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  uint32_t* stage = stage_all[threadIdx.x >> 6];
  const uint16_t* yr = y + row * N;
  const int nch = (int)(N / 8);
  uint4 raw[CPL];
#pragma unroll
  for (int u = 0; u < CPL; ++u)
    raw[u] = lane + 64 * u < nch ? *reinterpret_cast<const uint4*>(yr + 8 * (lane + 64 * u)) : make_uint4(0, 0, 0, 0);
  const int64_t base = row_ptr[row];
  const int limit = (int)(row_ptr[row + 1] - base);        // the row's room in cols / vals
  int32_t* cols_row = cols + base;
  uint16_t* vals_row = vals + base;
  int running = 0;
#pragma unroll
  for (int u = 0; u < CPL; ++u) {
    const int c = lane + 64 * u;
    float v[8];
    unpack8(raw[u], v);
    uint32_t m = 0;
    if (c < nch) {
#pragma unroll
      for (int j = 0; j < 8; ++j) m |= (v[j] > thr) ? (1u << j) : 0u;
    }
    const int cnt = __popc(m);
    const int incl = wave_inclusive_scan(cnt);
    int pos = running + incl - cnt;
    if (m) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if ((m >> j) & 1u) {
          stage_entry(stage, pos, limit, 8 * c + j, f_to_bf(v[j]), cols_row, vals_row);
          ++pos;
        }
      }
    }
    running += __builtin_amdgcn_readlane(incl, 63);
  }
  stage_flush(stage, running, limit, cols_row, vals_row);
}

// one wave per row; the output row is assembled in LDS (zeros + kept entries) and written out coalesced.
// BWD: dx = (g - s) * yh with s = bf16(sum_j bf16(g_j * yh_j)), every product rounded to bf16 as torch does.
template <bool BWD>
__global__ void __launch_bounds__(256)
k_softmax_rows(const uint16_t* g, int64_t rows, int64_t N, const int32_t* __restrict__ row_ptr,
               const int32_t* __restrict__ cols, const uint16_t* __restrict__ vals, uint16_t* out) {   // out may be g
  extern __shared__ __align__(16) uint16_t lds[];          // [4][N]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  uint16_t* buf = lds + (int64_t)wave * N;
  const int e0 = row_ptr[row], e1 = row_ptr[row + 1];
  float s = 0.f;
  if (BWD) {
    float part = 0.f;
    for (int e = e0 + lane; e < e1; e += 64)
      part += bfr(bf_to_f(g[row * N + cols[e]]) * bf_to_f(vals[e]));
    s = bfr(wave_sum(part));
  }
  for (int64_t c = lane; c < N / 8; c += 64) *reinterpret_cast<uint4*>(buf + 8 * c) = make_uint4(0, 0, 0, 0);
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // order this wave's LDS writes (other lanes) before the next ones
  __builtin_amdgcn_wave_barrier();
  for (int e = e0 + lane; e < e1; e += 64) {
    const int col = cols[e];
    const float yh = bf_to_f(vals[e]);
    buf[col] = BWD ? f_to_bf(bfr(bf_to_f(g[row * N + col]) - s) * yh) : vals[e];
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // the row leaves through streaming stores (written once, not read again here).  (Bringing the row of g in once, in
  // 16-byte pieces, for the kept entries to pick from a second LDS row was 3 % slower at 2048 entries and 20 % at 8192.)
  uint16_t* orow = out + row * N;
  for (int64_t c = lane; c < N / 8; c += 64) store_stream(orow + 8 * c, *reinterpret_cast<const uint4*>(buf + 8 * c));
}

static int softmax_shape(const char* who, int64_t rows, int64_t N) {
  if (rows < 0 || N <= 0 || N % 8 != 0 || N > 8192)
    return fail(rows < 0 || N <= 0 ? HYC_EINVAL : HYC_ENOTSUP, "%s: rows=%lld N=%lld (N must be a multiple of 8, at most 8192)",
                who, (long long)rows, (long long)N);
  return HYC_OK;
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_softmax_fwd(const void* x, int64_t rows, int64_t N, float threshold, void* y, int32_t* counts, void* stream) {
  int rc = softmax_shape("hyc_softmax_fwd", rows, N);
  if (rc) return rc;
  if (rows == 0) return HYC_OK;
  if (!y) return fail(HYC_EFAULT, "hyc_softmax_fwd: null y");
  if ((x && !aligned16(x)) || !aligned16(y)) return fail(HYC_EINVAL, "hyc_softmax_fwd: x and y must be 16-byte aligned");
  hipStream_t st = begin_launch(stream);
  const float thr = round_to_bf16(threshold);
  if (x && N <= 4096) {
    const int cpl = (int)((N / 8 + 63) / 64);             // chunks per lane: 1..8
    // one row per wave: a capped grid whose waves loop over rows is 6-15 % slower (the dispatcher balances short waves better)
    const int64_t blocks = (rows + 3) / 4, cap = blocks;
    const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
#define HYC_SMW_F(C_, F_)                                                                                          \
  hipLaunchKernelGGL((k_softmax_fwd_wave<C_, false, F_>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(x), rows, N, \
                     thr, static_cast<uint16_t*>(y), counts, (int64_t)1)
#define HYC_SMW(C_) do { if ((C_) > 1 && N == 512 * (C_)) HYC_SMW_F(C_, true); else HYC_SMW_F(C_, false); } while (0)
    if (cpl <= 1) HYC_SMW(1); else if (cpl <= 2) HYC_SMW(2); else if (cpl <= 4) HYC_SMW(4); else HYC_SMW(8);
#undef HYC_SMW
#undef HYC_SMW_F
  } else if (x) {
    const int64_t cap = 256 * 8;
    hipLaunchKernelGGL(k_softmax_fwd, dim3((unsigned)(rows < cap ? rows : cap)), dim3(256), 0, st,
                       static_cast<const uint16_t*>(x), rows, N, thr, static_cast<uint16_t*>(y), counts);
  } else {
    if (!counts) return fail(HYC_EFAULT, "hyc_softmax_fwd: nothing to do (x and counts both null)");
    hipLaunchKernelGGL(k_softmax_count, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st,
                       static_cast<const uint16_t*>(y), rows, N, thr, counts);
  }
  return check_launch("hyc_softmax_fwd");
}

int hyc_softmax_causal_fwd(const void* x, int64_t rows, int64_t N, int64_t period, float threshold, void* y,
                           int32_t* counts, void* stream) {
  int rc = softmax_shape("hyc_softmax_causal_fwd", rows, N);
  if (rc) return rc;
  if (N > 4096) return fail(HYC_ENOTSUP, "hyc_softmax_causal_fwd: N=%lld (rows of at most 4096 entries)", (long long)N);
  if (period <= 0 || period > N)
    return fail(HYC_EINVAL, "hyc_softmax_causal_fwd: period=%lld must be in 1..N=%lld", (long long)period, (long long)N);
  if (rows == 0) return HYC_OK;
  if (!x || !y) return fail(HYC_EFAULT, "hyc_softmax_causal_fwd: null buffer");
  if (!aligned16(x) || !aligned16(y)) return fail(HYC_EINVAL, "hyc_softmax_causal_fwd: x and y must be 16-byte aligned");
  hipStream_t st = begin_launch(stream);
  const float thr = round_to_bf16(threshold);
  const int cpl = (int)((N / 8 + 63) / 64);
  const int64_t blocks = (rows + 3) / 4, cap = blocks;        // one row per wave, see hyc_softmax_fwd
  const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
#define HYC_SMC_F(C_, F_)                                                                                         \
  hipLaunchKernelGGL((k_softmax_fwd_wave<C_, true, F_>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(x), rows, N, \
                     thr, static_cast<uint16_t*>(y), counts, period)
#define HYC_SMC(C_) do { if ((C_) > 1 && N == 512 * (C_)) HYC_SMC_F(C_, true); else HYC_SMC_F(C_, false); } while (0)
  if (cpl <= 1) HYC_SMC(1); else if (cpl <= 2) HYC_SMC(2); else if (cpl <= 4) HYC_SMC(4); else HYC_SMC(8);
#undef HYC_SMC
#undef HYC_SMC_F
  return check_launch("hyc_softmax_causal_fwd");
}

int hyc_csr_offsets(const int32_t* counts, int64_t rows, int64_t capacity, int32_t* row_ptr, int64_t* total, void* stream) {
  if (rows < 0) return fail(HYC_EINVAL, "hyc_csr_offsets: rows=%lld", (long long)rows);
  if (!row_ptr || (rows > 0 && !counts)) return fail(HYC_EFAULT, "hyc_csr_offsets: null buffer");
  if (capacity < 0 || capacity > 0x7FFFFFFFll) capacity = 0x7FFFFFFFll;          // row_ptr is int32
  if (aligned16(counts) && aligned16(row_ptr))
    hipLaunchKernelGGL(k_csr_offsets<true>, dim3(1), dim3(OFFS_THREADS), 0, begin_launch(stream), counts, rows, capacity, row_ptr, total);
  else
    hipLaunchKernelGGL(k_csr_offsets<false>, dim3(1), dim3(OFFS_THREADS), 0, begin_launch(stream), counts, rows, capacity, row_ptr, total);
  return check_launch("hyc_csr_offsets");
}

int hyc_softmax_fill(const void* y, int64_t rows, int64_t N, float threshold, const int32_t* row_ptr, int32_t* cols,
                     void* vals, void* stream) {
  int rc = softmax_shape("hyc_softmax_fill", rows, N);
  if (rc) return rc;
  if (rows == 0) return HYC_OK;
  if (!y || !row_ptr) return fail(HYC_EFAULT, "hyc_softmax_fill: null buffer");
  if (!aligned16(y)) return fail(HYC_EINVAL, "hyc_softmax_fill: y must be 16-byte aligned");
  hipStream_t st = begin_launch(stream);
  const dim3 grid((unsigned)((rows + 3) / 4));
  const float thr = round_to_bf16(threshold);
#define HYC_SMF(C_)                                                                                          \
  hipLaunchKernelGGL((k_softmax_fill_wave<C_>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(y), rows, N, thr, \
                     row_ptr, cols, static_cast<uint16_t*>(vals))
  const int cpl = (int)((N / 8 + 63) / 64);
  if (cpl <= 1) HYC_SMF(1); else if (cpl <= 2) HYC_SMF(2); else if (cpl <= 4) HYC_SMF(4); else if (cpl <= 8) HYC_SMF(8);
  else
    hipLaunchKernelGGL(k_softmax_fill, grid, dim3(256), 0, st, static_cast<const uint16_t*>(y), rows, N, thr, row_ptr,
                       cols, static_cast<uint16_t*>(vals));
#undef HYC_SMF
  return check_launch("hyc_softmax_fill");
}

int hyc_softmax_bwd(const void* g, int64_t rows, int64_t N, const int32_t* row_ptr, const int32_t* cols,
                    const void* vals, void* dx, void* stream) {
  int rc = softmax_shape("hyc_softmax_bwd", rows, N);
  if (rc) return rc;
  if (rows == 0) return HYC_OK;
  if (!g || !row_ptr || !dx) return fail(HYC_EFAULT, "hyc_softmax_bwd: null buffer");
  if (!aligned16(dx)) return fail(HYC_EINVAL, "hyc_softmax_bwd: dx must be 16-byte aligned");
  hipLaunchKernelGGL((k_softmax_rows<true>), dim3((unsigned)((rows + 3) / 4)), dim3(256), (size_t)N * 8, begin_launch(stream),
                     static_cast<const uint16_t*>(g), rows, N, row_ptr, cols, static_cast<const uint16_t*>(vals),
                     static_cast<uint16_t*>(dx));
  return check_launch("hyc_softmax_bwd");
}

int hyc_softmax_dense(int64_t rows, int64_t N, const int32_t* row_ptr, const int32_t* cols, const void* vals,
                      void* y_hat, void* stream) {
  int rc = softmax_shape("hyc_softmax_dense", rows, N);
  if (rc) return rc;
  if (rows == 0) return HYC_OK;
  if (!row_ptr || !y_hat) return fail(HYC_EFAULT, "hyc_softmax_dense: null buffer");
  if (!aligned16(y_hat)) return fail(HYC_EINVAL, "hyc_softmax_dense: y_hat must be 16-byte aligned");
  hipLaunchKernelGGL((k_softmax_rows<false>), dim3((unsigned)((rows + 3) / 4)), dim3(256), (size_t)N * 8, begin_launch(stream),
                     static_cast<const uint16_t*>(nullptr), rows, N, row_ptr, cols, static_cast<const uint16_t*>(vals),
                     static_cast<uint16_t*>(y_hat));
  return check_launch("hyc_softmax_dense");
}

}  // extern "C"
