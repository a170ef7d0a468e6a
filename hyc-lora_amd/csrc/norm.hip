// RMSNorm forward fused with the compression of its input, and RMSNorm backward fused with the
// decompression.  A row lives in registers (x is read from HBM once); the next row's loads are issued before the
// current row is processed so that memory requests stay in flight during the arithmetic.
#include <atomic>
#include <stdlib.h>

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

// Sum of two values over the `nw` waves of one row slot with ONE barrier: partials go to a buffer that alternates
// with `parity`, so the next reduction never overwrites values a slower wave is still reading.
// red layout: [2 parities][slots][16 waves][2 values].
__device__ __forceinline__ void slot_sum2(float& a, float& b, float* red, int parity, int slot, int nslots, int wave_in_slot,
                                          int nw) {
  a = wave_sum(a);
  b = wave_sum(b);
  float* base = red + ((parity * nslots + slot) * 16) * 2;
  if ((threadIdx.x & 63) == 0) { base[2 * wave_in_slot] = a; base[2 * wave_in_slot + 1] = b; }
  __syncthreads();
  float ta = 0.f, tb = 0.f;
  for (int i = 0; i < nw; ++i) { ta += base[2 * i]; tb += base[2 * i + 1]; }
  a = ta; b = tb;
}

// ------------------------------------------------------------------------------------------------
// Fast paths (channel mode, every lane owns exactly one chunk per segment: CPS == blockDim.x, LPG known at
// compile time).  No per-lane predication, row-invariant data (weights, plan words) hoisted, pointers advanced
// instead of recomputed, next row prefetched under a uniform branch.
// ------------------------------------------------------------------------------------------------
template <bool WF32>
__device__ __forceinline__ void load_w8t(const void* w, int64_t col, float (&o)[8]) {
  if (WF32) {
    const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + col);
    const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + col + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    unpack8(*reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(w) + col), o);
  }
}

// sum over the waves of the workgroup, one barrier (alternating buffers, see slot_sum2)
__device__ __forceinline__ float block_sum1(float a, float (*red)[16], int parity, int wave, int nw) {
  a = wave_sum(a);
  if ((threadIdx.x & 63) == 0) red[parity][wave] = a;
  __syncthreads();
  float t = red[parity][0];
  for (int i = 1; i < nw; ++i) t += red[parity][i];
  return t;
}

// ---- rows staged through LDS -------------------------------------------------------------------------------------
// gfx950 can load 16 bytes per lane from memory straight into LDS (global_load_lds_dwordx4: lane i of a wave lands at
// the wave's LDS base + 16 i).  A wave uses that as a prefetch queue of its own: the incoming-gradient chunks of the
// rows it will process next wait in LDS, not in registers, so several rows can be in flight per wave at no cost in
// occupancy.  Every wave only ever reads what it requested itself, so no barrier guards the queue.
//
// Completion: vector memory operations of a wave complete in issue order.  The small per-row loads that go to
// registers (codes, scales, outlier values, rstd) are issued AFTER the queue entry of the same row, and a queue entry
// is read only after one of those registers has been used, so the compiler's own wait for that register covers the
// entry.  The LDS reads are written in assembly: a read the compiler can see would make it wait for EVERY outstanding
// load into the queue array (it cannot tell the stages apart), which would undo the prefetch.
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* gbl_void_ptr;
constexpr int RING_D = 3;                                             // rows per wave in the queue: being read, next, after next

__device__ __forceinline__ uint32_t lds_offset(const void* p) {
  return (uint32_t)(size_t)(__attribute__((address_space(3))) const char*)p;
}
// NSEG chunks of 16 bytes per lane, 1 KB apart, at LDS byte address `addr` (this lane's); `after` is any register
// whose load was issued after the queue entry: naming it here keeps this read behind the wait for it
template <int NSEG>
__device__ __forceinline__ void queue_read(uint32_t addr, uint32_t after, uint4 (&g)[NSEG]) {
  static_assert(NSEG == 1 || NSEG == 2 || NSEG == 4, "chunks per lane");
  u32x4_t a, b = {0, 0, 0, 0}, c = {0, 0, 0, 0}, d = {0, 0, 0, 0};
  if (NSEG == 4)
    asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\tds_read_b128 %2, %4 offset:2048\n\t"
                 "ds_read_b128 %3, %4 offset:3072\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d) : "v"(addr), "v"(after) : "memory");
  else if (NSEG == 2)
    asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:1024\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(a), "=&v"(b) : "v"(addr), "v"(after) : "memory");
  else
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(a) : "v"(addr), "v"(after) : "memory");
  const u32x4_t v[4] = {a, b, c, d};
#pragma unroll
  for (int i = 0; i < NSEG; ++i) g[i] = make_uint4(v[i].x, v[i].y, v[i].z, v[i].w);
}

// rows per wave in the forward kernel's queue: three, or two where three would not leave room (long rows of 2-bit codes)
constexpr int fwd_queue_depth(int maxt, int nseg) { return RING_D * maxt * nseg * 16 <= 128 * 1024 ? RING_D : 2; }

// LN: LayerNorm with the two-pass statistics of operators/efficient_layernorm.py:15-61 (mean = sum(x)/H, var =
// sum((x - mean)^2)/H, y = ((x - mean)*rstd)*w + b): the row is in registers, so the second pass costs one more
// workgroup reduction and no memory traffic.
template <int BITS, int LPGT, bool WF32, int MAXT, int RULE, bool LN>
__device__ __forceinline__ void
norm_fwd_fast_rows(const uint16_t* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias, float eps,
                   int64_t M, int64_t H, int CPS, const ChanArgs& ca, uint16_t* __restrict__ y, float* __restrict__ mean_out,
                   float* __restrict__ rstd_out, uint8_t* __restrict__ stored, uint16_t* __restrict__ vals,
                   uint16_t* __restrict__ scales) {
  constexpr int NSEG = Q<BITS>::NSEG;
  constexpr int D = fwd_queue_depth(MAXT, NSEG);                      // rows in the queue
  __shared__ float red[2][16];
  // dynamic LDS, D stages of blockDim.x * NSEG chunks: [stage][wave][segment][lane], x chunks on their way in
  extern __shared__ __align__(16) uint4 queue[];
  const int STAGE_B = (int)blockDim.x * NSEG * 16;                    // bytes of one queue stage of the workgroup
  const int c = threadIdx.x;
  const bool active = c < CPS;                                    // false only in the tail of the last wave
  const uint32_t SEG = (uint32_t)CPS * 8u;
  const float invH = 1.0f / (float)H;
  const int wave = __builtin_amdgcn_readfirstlane(c >> 6), nw = blockDim.x >> 6;
  const bool leader = active && (c & (LPGT - 1)) == 0;
  const int seg_groups = CPS >> ca.chunk_to_group_shift;          // scale groups per segment
  // Every memory instruction of the row loop is a buffer operation on a resource that spans one row (zero bytes for a
  // row past the end); lanes without data carry the offset NOWHERE.  Nothing is predicated or branched on.
  const uint32_t row_b = (uint32_t)H * 2u, seg_b = SEG * 2u;
  const uint32_t xo = active ? 16u * (uint32_t)c : NOWHERE;                                       // y: chunk c of segment 0
  // (the same for x on its way into the queue, except that lanes past the end of the row re-read its first chunk: a
  // load into LDS with some of its lanes out of range runs several times slower - measured - than one with all or none)
  const uint32_t qo = active ? 16u * (uint32_t)c : 0u;
  const uint32_t so = active ? 8u * (uint32_t)c : NOWHERE;                                        // packed word
  const uint32_t go = leader ? 2u * (uint32_t)(c >> ca.chunk_to_group_shift) : NOWHERE;           // group scale (leaders)
  const uint32_t ro = c == 0 ? 0u : NOWHERE;                                                      // rstd (one lane)
  const bool gather = active && c < ca.k;                         // thread c copies outlier channel idx[c] to vals
  const uint32_t gi = gather ? 2u * (uint32_t)ca.idx[c] : NOWHERE, vo = gather ? 2u * (uint32_t)c : NOWHERE;
  char* const qwave = reinterpret_cast<char*>(queue) + wave * (NSEG * 1024);
  const uint32_t qlane = lds_offset(queue) + (uint32_t)(wave * (NSEG * 1024)) + 16u * (uint32_t)(c & 63);

  uint32_t km[NSEG][4];                                            // AND masks that zero the outlier channels
  float wv[NSEG][8], bv[LN ? NSEG : 1][8];
  {
    uint32_t plan[NSEG];
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      plan[i] = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) { wv[i][j] = 0.f; if (LN) bv[LN ? i : 0][j] = 0.f; }
      if (active) {
        plan[i] = ca.plan[i * CPS + c];
        load_w8t<WF32>(w, (int64_t)i * SEG + 8 * c, wv[i]);
        if (LN && bias) load_w8t<WF32>(bias, (int64_t)i * SEG + 8 * c, bv[LN ? i : 0]);
      }
    }
    ChunkOutliers<NSEG> co;
    co.init(plan);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) co.keep_masks(i, km[i]);
  }
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  auto row_of = [&](const void* base, int64_t r, uint32_t bytes) __attribute__((always_inline)) {
    return make_rsrc(static_cast<const char*>(base) + r * (int64_t)bytes, r < M ? bytes : 0u);
  };
  // row r into queue stage `stage_b`
  auto request = [&](int64_t r, int stage_b) __attribute__((always_inline)) {
    const BufferRsrc rs_x = row_of(x, r, row_b);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) load_b128_to_lds(rs_x, qo + (uint32_t)i * seg_b, qwave + stage_b + i * 1024);
  };
  // The outlier channel this thread copies to vals[r, :] goes to a register.  It is requested after row r's queue
  // entry and before the next entry, so having used it vouches for row r's entry and for nothing younger (see above).
  auto request_outlier = [&](int64_t r) __attribute__((always_inline)) { return load_b16(row_of(x, r, row_b), gi); };
  // The compiler sizes each wait by the fewest memory operations that can have been issued since the load it waits
  // for, over every path to that point.  Entering the loop must therefore look like coming around it: the requests
  // made ahead of the loop are followed by as many stores as a loop iteration issues after its requests (here to
  // nowhere: dropped before they reach memory).  Without them the wait at the top of the loop would be sized for the
  // first row and would drain the queue on every row.
  request(row, 0);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t og = request_outlier(row);
  __builtin_amdgcn_sched_barrier(0);
  if (D > 2) request(row + stride, STAGE_B);
  {
    const BufferRsrc nothing = make_rsrc(x, 0u);
    store_b32(nothing, NOWHERE, 0u);                                 // stands for: rstd
    if (LN) store_b32(nothing, NOWHERE + 4u, 0u);                    // mean
    store_b64(nothing, NOWHERE + 8u, 0u, 0u);                        // the packed word
#pragma unroll
    for (int i = 0; i < NSEG; ++i) store_b16(nothing, NOWHERE + 2u * (i + 1), (uint16_t)0);   // NSEG scales
#pragma unroll
    for (int i = 0; i < NSEG; ++i) store_b128_stream(nothing, NOWHERE + 16u * (i + 1), make_uint4(0, 0, 0, 0));   // NSEG chunks of y
    // (distinct offsets: identical stores would be folded into one)
  }
  __builtin_amdgcn_sched_barrier(0);
  int st_b = 0, parity = 0;
  for (; row < M; row += stride, parity ^= 1) {
    uint4 raw[NSEG];
    queue_read<NSEG>(qlane + (uint32_t)st_b, og, raw);
    const BufferRsrc rs_s = row_of(stored, row, SEG), rs_c = row_of(scales, row, 2u * (uint32_t)ca.groups_per_row);
    const BufferRsrc rs_v = row_of(vals, row, 2u * (uint32_t)ca.k);
    // the row's outlier value leaves at once and the next row's takes the register; then the row after next (two
    // ahead; one with a short queue) goes into the stage that was read one row ago
    store_b16(rs_v, vo, (uint16_t)og);
    __builtin_amdgcn_sched_barrier(0);
    if (D > 2) {
      og = request_outlier(row + stride);
      __builtin_amdgcn_sched_barrier(0);
      request(row + (D - 1) * stride, st_b >= STAGE_B ? st_b - STAGE_B : st_b + (D - 1) * STAGE_B);
    } else {
      // a queue of two: the next row's entry is requested here, so it has to be older than the register that will
      // vouch for it (with three stages that entry went out one row earlier)
      request(row + stride, st_b >= STAGE_B ? st_b - STAGE_B : st_b + STAGE_B);
      __builtin_amdgcn_sched_barrier(0);
      og = request_outlier(row + stride);
    }
    __builtin_amdgcn_sched_barrier(0);
    float ss = 0.f;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float v[8];
      unpack8(raw[i], v);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = LN ? ss + v[j] : __builtin_fmaf(v[j], v[j], ss);
      unpack8(make_uint4(raw[i].x & km[i][0], raw[i].y & km[i][1], raw[i].z & km[i][2], raw[i].w & km[i][3]), v);
      uint32_t cl, ch;
      const float s = quant_seg<BITS, LPGT, RULE>(v, LPGT, cl, ch, false);
      store_b16(rs_c, go + 2u * (uint32_t)(i * seg_groups), f_to_bf(s));
      if (BITS == 8) { lo = cl; hi = ch; }
      else { lo |= cl << (i * BITS); hi |= ch << (i * BITS); }
    }
    store_b64(rs_s, so, lo, hi);
    if (ca.k > CPS) {                                               // more outlier channels than threads (uniform, rare)
      const uint16_t* xrow = x + row * H;
      for (int t = c + CPS; t < ca.k; t += CPS) vals[row * ca.k + t] = xrow[ca.idx[t]];
    }
    // sum over the waves of the workgroup: one bare barrier (__syncthreads() would also wait for the loads on their way
    // into the queue), alternating buffers so that the next row's partial sums never overwrite values still being read
    // (lanes past the end of the row hold a copy of its first chunk: they stay out of the sum, and what they encode is
    // stored nowhere; scale groups never straddle the end of a row)
    ss = wave_sum(active ? ss : 0.f);
    if ((c & 63) == 0) red[parity][wave] = ss;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float tot = red[parity][0];
    for (int i = 1; i < nw; ++i) tot += red[parity][i];
    float mean = 0.f;
    if (LN) {
      // second pass over the registers; its partial sums take the other buffer (a wave can only write that one again
      // after the next row's first barrier, which every wave reaches after it has read this row's values)
      mean = tot * invH;
      float var = 0.f;
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float v[8];
        unpack8(raw[i], v);
#pragma unroll
        for (int j = 0; j < 8; ++j) { const float dlt = v[j] - mean; var = __builtin_fmaf(dlt, dlt, var); }
      }
      parity ^= 1;
      var = wave_sum(active ? var : 0.f);
      if ((c & 63) == 0) red[parity][wave] = var;
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      tot = red[parity][0];
      for (int i = 1; i < nw; ++i) tot += red[parity][i];
      store_b32(row_of(mean_out, row, 4u), ro, __float_as_uint(mean));
    }
    const float rstd = 1.0f / __builtin_sqrtf(tot * invH + eps);
    store_b32(row_of(rstd_out, row, 4u), ro, __float_as_uint(rstd));
    const BufferRsrc rs_y = row_of(y, row, row_b);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float v[8];
      unpack8(raw[i], v);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = LN ? ((v[j] - mean) * rstd) * wv[i][j] + bv[LN ? i : 0][j] : (v[j] * rstd) * wv[i][j];
      store_b128_stream(rs_y, xo + (uint32_t)i * seg_b, pack8(v));
    }
    st_b = st_b >= (D - 1) * STAGE_B ? 0 : st_b + STAGE_B;
  }
}

template <int BITS, int LPGT, bool WF32, int MAXT, int RULE>
__global__ void __launch_bounds__(MAXT)
k_rmsnorm_fwd_fast(const uint16_t* __restrict__ x, const void* __restrict__ w, float eps, int64_t M, int64_t H,
                   int CPS, ChanArgs ca, uint16_t* __restrict__ y, float* __restrict__ rstd_out, uint8_t* __restrict__ stored,
                   uint16_t* __restrict__ vals, uint16_t* __restrict__ scales) {
  norm_fwd_fast_rows<BITS, LPGT, WF32, MAXT, RULE, false>(x, w, nullptr, eps, M, H, CPS, ca, y, nullptr, rstd_out, stored, vals, scales);
}

template <int BITS, int LPGT, bool WF32, int MAXT, int RULE>
__global__ void __launch_bounds__(MAXT)
k_layernorm_fwd_fast(const uint16_t* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias, float eps,
                     int64_t M, int64_t H, int CPS, ChanArgs ca, uint16_t* __restrict__ y, float* __restrict__ mean_out,
                     float* __restrict__ rstd_out, uint8_t* __restrict__ stored, uint16_t* __restrict__ vals,
                     uint16_t* __restrict__ scales) {
  norm_fwd_fast_rows<BITS, LPGT, WF32, MAXT, RULE, true>(x, w, bias, eps, M, H, CPS, ca, y, mean_out, rstd_out, stored, vals, scales);
}

// two float4 at LDS byte addresses `addr` and `addr + second`
__device__ __forceinline__ void lds_read_8f(uint32_t addr, uint32_t second, float (&o)[8]) {
  floatx4_t a, b;
  asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %3\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b) : "v"(addr), "v"(addr + second) : "memory");
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

// Backward fast path.  A workgroup is `slots` row slots of CPS threads; slot s of workgroup b handles rows
// b*slots + s, + gridDim.x*slots, ...: the rows in flight across the chip are adjacent in memory (rows that are far
// apart would crowd onto a few memory channels).  Each slot keeps its own dw accumulators; they are added through
// LDS at the end, in slot order, so a workgroup writes one fp32 partial row.
// DENSE: `stored` is the restored activation itself (bf16 [M, H]; what a threshold-scheme caller hands over after
// hyc_decompress), read with the chunk mapping of 4-bit codes; nothing is decoded.
// D: rows per wave in the queue (three; two for rows so long that the weight row leaves no room for a third stage)
template <int BITS, bool WF32, bool QUIRK, int MAXT, bool DENSE, int D>
__device__ __forceinline__ void
norm_bwd_fast_rows(const uint16_t* __restrict__ dy, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
                   const uint16_t* __restrict__ scales, const void* __restrict__ w, const float* __restrict__ rstd,
                   const float* __restrict__ mean, int64_t M, int64_t H, int T, int CPS, int slots, int steps, ChanArgs ca,
                   uint16_t* __restrict__ dx, float* __restrict__ dw_partials) {
  // A thread decodes at most two segments of its packed word: with four segments (2-bit codes) two threads share
  // a word, which keeps the per-thread state (and so the occupancy) the same for every bit width.
  constexpr int NSEG = Q<BITS>::NSEG > 2 ? 2 : Q<BITS>::NSEG;         // segments per thread
  constexpr int PARTS = Q<BITS>::NSEG / NSEG;                         // threads per packed word
  constexpr int STAGE_B = MAXT * NSEG * 16;                           // bytes of one queue stage of the workgroup
  __shared__ float red[2][4][2][16];                                  // [parity][slot][value][wave]
  __shared__ __align__(16) uint4 queue[D * MAXT * NSEG];              // [stage][wave][segment][lane]: dy chunks on their way in
  // dynamic LDS: the weight row as fp32 [segment][half chunk][CPS] float4 (read again for every row: sixteen
  // registers fewer than keeping the thread's weights live)
  extern __shared__ __align__(16) float lds_dyn[];
  float4* wl4 = reinterpret_cast<float4*>(lds_dyn);
  // T = PARTS*CPS rounded up to whole waves, so the slot is the same for a whole wave: row bases stay scalar
  // (at most four slots and two threads per packed word: comparisons instead of integer divisions)
  const int tid_u = __builtin_amdgcn_readfirstlane((int)threadIdx.x & ~63);
  const int slot = (tid_u >= T) + (tid_u >= 2 * T) + (tid_u >= 3 * T);
  const int u = (int)threadIdx.x - slot * T;
  const bool active = u < PARTS * CPS;
  const int part = (PARTS > 1 && u >= CPS) ? 1 : 0, c = u - part * CPS;
  static_assert(PARTS <= 2, "two threads per packed word at most");
  const int seg0 = part * NSEG;                                       // first segment of this thread
  const int SEG = CPS * 8;                                            // channels per segment = bytes per stored row
  const float invH = 1.0f / (float)H;
  const int wave = u >> 6, nw = T >> 6;
  const int seg_groups = CPS >> ca.chunk_to_group_shift;
  // Byte offsets of the thread inside a row of each tensor.  Every memory instruction of the row loop is a buffer
  // operation on a resource that spans one row (zero bytes for a row past the end), and lanes past the end of the
  // row (the tail of a slot's last wave) carry the offset NOWHERE: nothing is predicated or branched on.
  const uint32_t xo = active ? (uint32_t)(seg0 * SEG + 8 * c) * 2u : NOWHERE;
  // (into the queue, lanes past the end of the row re-read its first chunk: a load into LDS with some of its lanes out
  // of range runs several times slower - measured - than one with all or none; what they read is zeroed below)
  const uint32_t qo = active ? xo : 0u;
  const uint32_t so = active ? 8u * (uint32_t)c : NOWHERE;
  const uint32_t go = active ? (uint32_t)(seg0 * seg_groups + (c >> ca.chunk_to_group_shift)) * 2u : NOWHERE;
  const uint32_t seg_b = (uint32_t)SEG * 2u, grp_b = (uint32_t)seg_groups * 2u;
  const uint32_t row_b = (uint32_t)H * 2u, sc_b = (uint32_t)ca.groups_per_row * 2u, val_b = (uint32_t)ca.k * 2u;
  // the wave's place in a queue stage, and this lane's
  const int wv = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  char* const qwave = reinterpret_cast<char*>(queue) + wv * (NSEG * 1024);
  const uint32_t qlane = lds_offset(queue) + (uint32_t)(wv * (NSEG * 1024)) + 16u * (threadIdx.x & 63);

  const uint32_t wl_lane = lds_offset(wl4) + (active ? (uint32_t)(seg0 * 2 * CPS + c) : 0u) * 16u;   // this thread's weights in LDS
  const int64_t stride = (int64_t)gridDim.x * slots;
  int64_t row = (int64_t)blockIdx.x * slots + slot;
  // (steps = ceil(M / stride), the same for every slot so that barriers stay matched; divided on the host)
  // row r of a tensor whose rows are `bytes` long, as a resource; empty when the row does not exist
  auto row_of = [&](const void* base, int64_t r, uint32_t bytes) __attribute__((always_inline)) {
    return make_rsrc(static_cast<const char*>(base) + r * (int64_t)bytes, r < M ? bytes : 0u);
  };
  // the dy chunks of row r into queue stage `stage_b` (a byte offset)
  auto request_dy = [&](int64_t r, int stage_b) __attribute__((always_inline)) {
    const BufferRsrc rs_g = row_of(dy, r, row_b);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) load_b128_to_lds(rs_g, qo + (uint32_t)i * seg_b, qwave + stage_b + i * 1024);
  };

  uint2 pk = make_uint2(0, 0);
  uint4 xraw[NSEG];                                                   // DENSE: the activation chunks of this row
  uint32_t sc[NSEG];   // one register each: a packed pair would be assembled right after the load and stall on it
  uint32_t o0[NSEG], o1[NSEG];
  uint32_t vo0[NSEG], vo1[NSEG];                                      // offsets of the chunk's first two outlier values
  float rs = 0.f, mu = 0.f;                                           // mu: LayerNorm's row mean (0 for RMSNorm)
  const uint16_t* vrow = vals;                                        // outlier values of the current row
  // the small operands of row r, to registers: codes, scales, rstd ...
  auto request_codes = [&](int64_t r) __attribute__((always_inline)) {
    // (vector loads although rstd is the same for the whole slot: a scalar load in flight would turn every wait for
    // an LDS read into a wait for it, too)
    rs = __uint_as_float(load_b32(row_of(rstd, r, 4u), 0u));
    if (mean) mu = __uint_as_float(load_b32(row_of(mean, r, 4u), 0u));
    if (DENSE) {
      const BufferRsrc rs_x = row_of(stored, r, row_b);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) xraw[i] = load_b128(rs_x, xo + (uint32_t)i * seg_b);
    } else {
      pk = load_b64(row_of(stored, r, (uint32_t)SEG), so);
      const BufferRsrc rs_c = row_of(scales, r, sc_b);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) sc[i] = load_b16(rs_c, go + (uint32_t)i * grp_b);
    }
  };
  // ... and the chunk's first two outlier values (needs the selectors)
  auto request_outliers = [&](int64_t r) __attribute__((always_inline)) {
    if (!DENSE) {
      const BufferRsrc rs_v = row_of(vals, r, val_b);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) { o0[i] = load_b16(rs_v, vo0[i]); o1[i] = load_b16(rs_v, vo1[i]); }
      vrow = vals + (r < M ? r : M - 1) * ca.k;
    }
  };

  // What the row loop needs first is asked for first: the thread's plan words and (first slot) its weights; then the
  // first two rows of dy and the first row's codes, which travel while the plan is turned into selectors and the
  // weight row goes to LDS; the first row's outlier values last (their place follows from the selectors).  Row 0's
  // registers are requested after row 0's queue entry, see above (row 1's entry is older too, so the first row waits
  // for both; they were requested together).
  uint32_t plan[NSEG];
  float acc[NSEG][8], wv8[NSEG][8];
#pragma unroll
  for (int i = 0; i < NSEG; ++i) {
    plan[i] = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) { acc[i][j] = 0.f; wv8[i][j] = 0.f; }
    if (active) {
      if (!DENSE) plan[i] = ca.plan[(seg0 + i) * CPS + c];
      if (slot == 0) load_w8t<WF32>(w, (int64_t)(seg0 + i) * SEG + 8 * c, wv8[i]);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  request_dy(row, 0);
  if (D > 2) request_dy(row + stride, STAGE_B);
  __builtin_amdgcn_sched_barrier(0);
  request_codes(row);
  __builtin_amdgcn_sched_barrier(0);
  if (active && slot == 0) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      wl4[((seg0 + i) * 2 + 0) * CPS + c] = make_float4(wv8[i][0], wv8[i][1], wv8[i][2], wv8[i][3]);
      wl4[((seg0 + i) * 2 + 1) * CPS + c] = make_float4(wv8[i][4], wv8[i][5], wv8[i][6], wv8[i][7]);
    }
  }
  ChunkOutliers<NSEG> co;
  co.init(plan);
#pragma unroll
  for (int i = 0; i < NSEG; ++i) {
    vo0[i] = co.has0[i] ? co.vb[i] : NOWHERE;
    vo1[i] = co.has1[i] ? co.vb[i] + 2u : NOWHERE;
  }
  request_outliers(row);
  __builtin_amdgcn_sched_barrier(0);
  // The compiler sizes each wait by the fewest memory operations that can have been issued since the load it waits
  // for, over every path to that point.  In the loop a row's registers are followed by a queue request and the
  // previous row's stores; entering the loop must look the same, or the waits at the top of the loop would be sized
  // for the first row and drain the queue on every row.  So: a request for a row past the end (zeros into the stage
  // that the first iteration requests next) and as many stores to nowhere (dropped before they reach memory).
  if (D > 2) request_dy(M, (D - 1) * STAGE_B);
#pragma unroll
  for (int i = 0; i < NSEG; ++i)   // (distinct offsets: identical stores would be folded into one)
    store_b128_stream(make_rsrc(dx, 0u), NOWHERE + 16u * i, make_uint4(0, 0, 0, 0));
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // the weight row is in LDS (no wait for the queue)
  int st_b = 0;                                                       // queue stage of the current row, as a byte offset
  int parity = 0;
  for (int step = 0; step < steps; ++step, row += stride, parity ^= 1) {
    float xn[NSEG][8], wdy[NSEG][8];
    float p1 = 0.f, p2 = 0.f;
    const float rs_c = rs;
    {
      // (a row past the end, and lanes past the end of a row, have read zeros for every operand - queue entries
      // included - so they add exact zeros to the sums below: no branch, no selects)
      const float nm = -mu * rs;                                      // xn = (x_hat - mean) * rstd as one fma
      uint4 graw[NSEG];
      queue_read<NSEG>(qlane + (uint32_t)st_b, DENSE ? xraw[0].x : sc[0], graw);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float g[8];
        unpack8(graw[i], g);
        if (DENSE) {
          unpack8(xraw[i], xn[i]);
        } else {
          // dx and dw are compared to a tolerance: the lean decode (scales of 1e30 and beyond and the sign of a zero
          // outlier are not its concern)
          uint4 r = co.splice_value(i, dequant8_fast<BITS>(pk.x, pk.y, seg0 + i, bf_to_f((uint16_t)sc[i])), o0[i], o1[i]);
          if (co.more_pairs) r = splice_more(r, co.more_pairs, ca.plan[(seg0 + i) * CPS + c], vrow, active, 1.f);
          unpack8(r, xn[i]);
        }
        // the thread's weights, re-read per row (sixteen registers fewer than keeping them live); in assembly for the
        // same reason as the queue reads: a read of dynamic LDS that the compiler can see waits for the queue to drain
        float wv[8];
        lds_read_8f(wl_lane + (uint32_t)(i * 2 * CPS) * 16u, (uint32_t)CPS * 16u, wv);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float n = __builtin_fmaf(xn[i][j], rs, nm);
          const float t = wv[j] * g[j];
          xn[i][j] = n;
          wdy[i][j] = t;
          p1 = __builtin_fmaf(n, t, p1);
          if (QUIRK) p2 += t;
          acc[i][j] = __builtin_fmaf(g[j], n, acc[i][j]);
        }
      }
      // (lanes past the end of the row hold the row's first chunk of dy and weights: they stay out of the row sums;
      // their dw sums are never stored)
      p1 = active ? p1 : 0.f;
      if (QUIRK) p2 = active ? p2 : 0.f;
    }
    // The row is decoded: its registers take the next row's codes, scales and outliers now, and the row after that
    // goes into the queue stage that was read two rows ago.  Order matters, see above.
    __builtin_amdgcn_sched_barrier(0);
    if (D == 2) {
      // a queue of two: the next row's entry takes the stage that was just read, and it must be OLDER than the next
      // row's registers, whose use vouches for it
      request_dy(row + stride, st_b >= STAGE_B ? st_b - STAGE_B : st_b + STAGE_B);
      __builtin_amdgcn_sched_barrier(0);
    }
    request_codes(row + stride);
    request_outliers(row + stride);
    __builtin_amdgcn_sched_barrier(0);
    if (D > 2) request_dy(row + (D - 1) * stride, st_b >= STAGE_B ? st_b - STAGE_B : st_b + (D - 1) * STAGE_B);
    __builtin_amdgcn_sched_barrier(0);
    // two sums per slot, one barrier
    p1 = wave_sum(p1);
    if (QUIRK) p2 = wave_sum(p2);
    if ((u & 63) == 0) { red[parity][slot][0][wave] = p1; if (QUIRK) red[parity][slot][1][wave] = p2; }
    // a bare barrier: __syncthreads() would also wait for every load on its way into the queue
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float t1 = red[parity][slot][0][0], t2 = QUIRK ? red[parity][slot][1][0] : 0.f;
    for (int i = 1; i < nw; ++i) { t1 += red[parity][slot][0][i]; if (QUIRK) t2 += red[parity][slot][1][i]; }
    // dx = (wdy - (xn*c1 + c2)) * rstd, arranged as two fused multiply-adds
    const float k1 = -(t1 * invH) * rs_c;
    const float k2 = QUIRK ? -(t2 * invH) * rs_c : 0.f;
    const BufferRsrc rs_o = row_of(dx, row, row_b);
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = __builtin_fmaf(xn[i][j], k1, __builtin_fmaf(wdy[i][j], rs_c, k2));
      store_b128_stream(rs_o, xo + (uint32_t)i * seg_b, pack8(o));
    }
    st_b = st_b >= (D - 1) * STAGE_B ? 0 : st_b + STAGE_B;
  }
  // The slots' dw sums are added in slot order through the queue's memory, which nobody reads any more.
  float* pr = dw_partials + (int64_t)blockIdx.x * H + (int64_t)seg0 * SEG + 8 * c;
  if (slots > 1) {
    float4* xs = reinterpret_cast<float4*>(queue);                     // [slots-1][T][NSEG][2] float4
    __syncthreads();
    if (slot > 0) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float4* o = xs + (((int64_t)(slot - 1) * T + u) * NSEG + i) * 2;
        o[0] = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
        o[1] = make_float4(acc[i][4], acc[i][5], acc[i][6], acc[i][7]);
      }
    }
    __syncthreads();
    if (slot == 0) {
      for (int s2 = 1; s2 < slots; ++s2) {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          const float4* o = xs + (((int64_t)(s2 - 1) * T + u) * NSEG + i) * 2;
          const float4 a = o[0], b = o[1];
          acc[i][0] += a.x; acc[i][1] += a.y; acc[i][2] += a.z; acc[i][3] += a.w;
          acc[i][4] += b.x; acc[i][5] += b.y; acc[i][6] += b.z; acc[i][7] += b.w;
        }
      }
    }
  }
  if (slot == 0 && active) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      float4* o = reinterpret_cast<float4*>(pr + (int64_t)i * SEG);
      o[0] = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
      o[1] = make_float4(acc[i][4], acc[i][5], acc[i][6], acc[i][7]);
    }
  }
}

#define HYC_NORM_BWD_FAST_PARAMS                                                                                      \
  const uint16_t* __restrict__ dy, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,              \
  const uint16_t* __restrict__ scales, const void* __restrict__ w, const float* __restrict__ rstd,                     \
  const float* __restrict__ mean, int64_t M, int64_t H, int T, int CPS, int slots, int steps, ChanArgs ca,             \
  uint16_t* __restrict__ dx, float* __restrict__ dw_partials
template <int BITS, bool WF32, bool QUIRK, int MAXT, bool DENSE = false>
__global__ void __launch_bounds__(MAXT) __attribute__((amdgpu_waves_per_eu(4, 8)))
k_rmsnorm_bwd_fast(HYC_NORM_BWD_FAST_PARAMS) {
  norm_bwd_fast_rows<BITS, WF32, QUIRK, MAXT, DENSE, RING_D>(dy, stored, vals, scales, w, rstd, mean, M, H, T, CPS, slots, steps, ca,
                                                              dx, dw_partials);
}
// rows of 1024 chunks per segment (16 384 channels of 4-bit codes): a queue of two stages beside the 64 KB weight row
template <int BITS, bool WF32, bool QUIRK>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 8)))
k_rmsnorm_bwd_fast_long(HYC_NORM_BWD_FAST_PARAMS) {
  norm_bwd_fast_rows<BITS, WF32, QUIRK, 1024, false, 2>(dy, stored, vals, scales, w, rstd, mean, M, H, T, CPS, slots, steps, ca,
                                                        dx, dw_partials);
}
#undef HYC_NORM_BWD_FAST_PARAMS

// ------------------------------------------------------------------------------------------------
// forward: y, rstd, and x compressed.  MODE 0 = channel, 1 = threshold.  One workgroup = one row at a time.
// LN: LayerNorm instead of RMSNorm, with the two-pass statistics of operators/efficient_layernorm.py:15-61
// (mean = sum(x)/H, var = sum((x - mean)^2)/H, y = ((x - mean)*rstd)*w + b); the row is in registers, so the
// second pass costs one more workgroup reduction and no memory traffic.
// ------------------------------------------------------------------------------------------------
template <int BITS, int ITERS, int MAXT, int MODE, bool LN = false>
__global__ void __launch_bounds__(MAXT)
k_rmsnorm_fwd(const uint16_t* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias, bool wf32,
              float eps, int64_t M, int64_t H,
              int CPS, ChanArgs ca, int lpg, ThrArgs ta, bool perchan, uint16_t* __restrict__ y,
              float* __restrict__ mean_out, float* __restrict__ rstd_out, uint8_t* __restrict__ stored,
              uint16_t* __restrict__ vals, uint16_t* __restrict__ scales, int32_t* __restrict__ row_counts) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ float red[2 * 16 * 2];
  const int64_t SEG = (int64_t)CPS * 8;
  const float invH = 1.0f / (float)H;
  const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;

  // what does not change from row to row: which chunks this thread owns and their outlier plan words
  bool act[ITERS];
  int cidx[ITERS];
  uint32_t plan[ITERS][NSEG];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    cidx[it] = it * blockDim.x + threadIdx.x;
    act[it] = cidx[it] < CPS;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) plan[it][i] = (MODE == 0 && act[it]) ? ca.plan[i * CPS + cidx[it]] : 0u;
  }

  uint4 raw[ITERS][NSEG];
  int64_t row = blockIdx.x;
  if (row < M) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int i = 0; i < NSEG; ++i)
        raw[it][i] = act[it] ? *reinterpret_cast<const uint4*>(x + row * H + i * SEG + 8 * cidx[it]) : make_uint4(0, 0, 0, 0);
  }
  int parity = 0;
  for (; row < M; row += gridDim.x, parity ^= 1) {
    // prefetch the next row
    uint4 nxt[ITERS][NSEG];
    const int64_t nrow = row + gridDim.x;
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int i = 0; i < NSEG; ++i)
        nxt[it][i] = (nrow < M && act[it]) ? *reinterpret_cast<const uint4*>(x + nrow * H + i * SEG + 8 * cidx[it])
                                           : make_uint4(0, 0, 0, 0);

    float ss = 0.f, hot = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = cidx[it];
      uint32_t lo = 0, hi = 0;
      if (MODE == 0) {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          float v[8];
          unpack8(raw[it][i], v);
#pragma unroll
          for (int j = 0; j < 8; ++j) ss = LN ? ss + v[j] : __builtin_fmaf(v[j], v[j], ss);
          uint32_t cl, ch;
          const float s = encode_seg<BITS>(raw[it][i], v, plan[it][i], lpg, vals + row * ca.k, cl, ch, ca.absmax != 0);
          if (act[it] && (c & (lpg - 1)) == 0)
            scales[row * ca.groups_per_row + ((i * CPS + c) >> ca.chunk_to_group_shift)] = f_to_bf(s);
          if (BITS == 8) { lo = cl; hi = ch; }
          else { lo |= cl << (i * BITS); hi |= ch << (i * BITS); }
        }
      } else {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          float v[8];
          unpack8(raw[it][i], v);
#pragma unroll
          for (int j = 0; j < 8; ++j) ss = LN ? ss + v[j] : __builtin_fmaf(v[j], v[j], ss);
        }
        if (act[it]) {
          hot += (float)(perchan ? encode_thr<BITS, true>(raw[it], c, CPS, H, row % ta.S, ta, lo, hi)
                                 : encode_thr<BITS, false>(raw[it], c, CPS, H, row % ta.S, ta, lo, hi));
        }
      }
      if (act[it]) *reinterpret_cast<uint2*>(stored + row * SEG + 8 * c) = make_uint2(lo, hi);
    }
    slot_sum2(ss, hot, red, parity, 0, 1, wave, nw);
    float mean = 0.f;
    if (LN) {
      mean = ss * invH;
      float var = 0.f, unused = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (act[it]) {                                  // lanes past the row hold zeros, not x - mean
#pragma unroll
          for (int i = 0; i < NSEG; ++i) {
            float v[8];
            unpack8(raw[it][i], v);
#pragma unroll
            for (int j = 0; j < 8; ++j) { const float dlt = v[j] - mean; var = __builtin_fmaf(dlt, dlt, var); }
          }
        }
      }
      parity ^= 1;                                      // the other buffer: see slot_sum2
      slot_sum2(var, unused, red, parity, 0, 1, wave, nw);
      ss = var;
    }
    const float rstd = 1.0f / __builtin_sqrtf(ss * invH + eps);
    if (threadIdx.x == 0) {
      rstd_out[row] = rstd;
      if (LN) mean_out[row] = mean;
      if (MODE == 1 && row_counts) row_counts[row] = (int32_t)hot;
    }
    uint16_t* yr = y + row * H;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      if (act[it]) {
#pragma unroll
        for (int i = 0; i < NSEG; ++i) {
          const int64_t col = i * SEG + 8 * cidx[it];
          float v[8], wv[8];
          unpack8(raw[it][i], v);
          load_w8(w, wf32, col, wv);
          if (LN) {
            float bv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) bv[j] = 0.f;
            if (bias) load_w8(bias, wf32, col, bv);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = ((v[j] - mean) * rstd) * wv[j] + bv[j];
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (v[j] * rstd) * wv[j];
          }
          *reinterpret_cast<uint4*>(yr + col) = pack8(v);
        }
      }
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int i = 0; i < NSEG; ++i) raw[it][i] = nxt[it][i];
  }
}

// ------------------------------------------------------------------------------------------------
// backward.  SRC 0 = channel-compressed x, 2 = dense bf16 x_hat.
// A workgroup is `slots` row slots of T threads; slot s handles rows r0+s, r0+s+slots, ... of the workgroup's
// range, keeps its own dw accumulators, and the slots are added up through LDS at the end (one fp32 partial row
// per workgroup).  All slots walk the same number of iterations so that they meet at the same barriers.
// ------------------------------------------------------------------------------------------------
template <int BITS, int ITERS, int MAXT, int SRC>
__global__ void __launch_bounds__(MAXT)
k_rmsnorm_bwd(const uint16_t* __restrict__ dy, const uint8_t* __restrict__ stored, const uint16_t* __restrict__ vals,
              const uint16_t* __restrict__ scales, const void* __restrict__ w, bool wf32,
              const float* __restrict__ rstd, const float* __restrict__ mean, int64_t M, int64_t H, int CPS, int T,
              int slots, int rows_per_block, ChanArgs ca, bool quirk, uint16_t* __restrict__ dx,
              float* __restrict__ dw_partials) {
  constexpr int NSEG = Q<BITS>::NSEG;
  __shared__ float red[2 * 16 * 16 * 2];
  extern __shared__ __align__(16) float xslot[];                        // [slots-1][T][8] for the final reduction
  const int64_t SEG = (int64_t)CPS * 8;
  const float invH = 1.0f / (float)H;
  const int slot = threadIdx.x / T, tl = threadIdx.x - slot * T;
  const int wave_in_slot = tl >> 6, nw = T >> 6;

  bool act[ITERS];
  int cidx[ITERS];
  uint32_t plan[ITERS][NSEG];
  float wv[ITERS][NSEG][8], acc[ITERS][NSEG][8];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    cidx[it] = it * T + tl;
    act[it] = cidx[it] < CPS;
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      plan[it][i] = (SRC == 0 && act[it]) ? ca.plan[i * CPS + cidx[it]] : 0u;
      if (act[it]) load_w8(w, wf32, i * SEG + 8 * cidx[it], wv[it][i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) { acc[it][i][j] = 0.f; if (!act[it]) wv[it][i][j] = 0.f; }
    }
  }

  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = r0 + rows_per_block < M ? r0 + rows_per_block : M;
  const int steps = (rows_per_block + slots - 1) / slots;

  // per-row inputs, loaded one step ahead
  uint2 pk[ITERS];
  uint4 graw[ITERS][NSEG];
  uint4 xraw[ITERS][NSEG];        // SRC 2 only
  uint16_t sc[ITERS][NSEG];       // SRC 0 only
  float rs = 0.f;
  auto load_row = [&](int64_t row, uint2 (&pk_)[ITERS], uint4 (&g_)[ITERS][NSEG], uint4 (&x_)[ITERS][NSEG],
                      uint16_t (&sc_)[ITERS][NSEG], float& rs_) {
    const bool valid = row < r1;
    rs_ = valid ? rstd[row] : 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const bool on = valid && act[it];
      if (SRC == 0) pk_[it] = on ? *reinterpret_cast<const uint2*>(stored + row * SEG + 8 * cidx[it]) : make_uint2(0, 0);
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        const int64_t col = i * SEG + 8 * cidx[it];
        g_[it][i] = on ? *reinterpret_cast<const uint4*>(dy + row * H + col) : make_uint4(0, 0, 0, 0);
        if (SRC == 0) {
          sc_[it][i] = on ? scales[row * ca.groups_per_row + ((i * CPS + cidx[it]) >> ca.chunk_to_group_shift)] : (uint16_t)0;
        } else {
          x_[it][i] = on ? *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(stored) + row * H + col)
                         : make_uint4(0, 0, 0, 0);
        }
      }
    }
  };
  load_row(r0 + slot, pk, graw, xraw, sc, rs);

  int parity = 0;
  for (int step = 0; step < steps; ++step, parity ^= 1) {
    const int64_t row = r0 + (int64_t)step * slots + slot;
    const bool valid = row < r1;
    uint2 pk_n[ITERS];
    uint4 g_n[ITERS][NSEG], x_n[ITERS][NSEG];
    uint16_t sc_n[ITERS][NSEG];
    float rs_n;
    load_row(row + slots, pk_n, g_n, x_n, sc_n, rs_n);

    float xn[ITERS][NSEG][8];
    float p1 = 0.f, p2 = 0.f;
    const float nm = (mean && valid) ? -mean[row] * rs : 0.f;        // LayerNorm: xn = (x_hat - mean) * rstd as one fma
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
#pragma unroll
      for (int i = 0; i < NSEG; ++i) {
        float g[8];
        unpack8(graw[it][i], g);
        if (SRC == 0) {
          unpack8(decode_seg<BITS>(pk[it].x, pk[it].y, i, bf_to_f(sc[it][i]), valid ? plan[it][i] : 0u, vals + row * ca.k),
                  xn[it][i]);
        } else {
          unpack8(xraw[it][i], xn[it][i]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float n = __builtin_fmaf(xn[it][i][j], rs, nm);
          const float t = wv[it][i][j] * g[j];
          xn[it][i][j] = n;
          p1 = __builtin_fmaf(n, t, p1);
          if (quirk) p2 += t;
          acc[it][i][j] = __builtin_fmaf(g[j], n, acc[it][i][j]);
        }
      }
    }
    slot_sum2(p1, p2, red, parity, slot, slots, wave_in_slot, nw);
    const float c1 = p1 * invH;
    const float c2 = quirk ? p2 * invH : 0.f;
    if (valid) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (act[it]) {
#pragma unroll
          for (int i = 0; i < NSEG; ++i) {
            float o[8], g[8];
            unpack8(graw[it][i], g);
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (wv[it][i][j] * g[j] - __builtin_fmaf(xn[it][i][j], c1, c2)) * rs;
            *reinterpret_cast<uint4*>(dx + row * H + i * SEG + 8 * cidx[it]) = pack8(o);
          }
        }
      }
    }
    rs = rs_n;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      pk[it] = pk_n[it];
#pragma unroll
      for (int i = 0; i < NSEG; ++i) { graw[it][i] = g_n[it][i]; xraw[it][i] = x_n[it][i]; sc[it][i] = sc_n[it][i]; }
    }
  }

  // add the slots' accumulators (slot order) and write the workgroup's partial row
  float* pr = dw_partials + (int64_t)blockIdx.x * H;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
#pragma unroll
    for (int i = 0; i < NSEG; ++i) {
      if (slots > 1) {
        __syncthreads();
        if (slot > 0) {
          float4* o = reinterpret_cast<float4*>(xslot + ((int64_t)(slot - 1) * T + tl) * 8);
          o[0] = make_float4(acc[it][i][0], acc[it][i][1], acc[it][i][2], acc[it][i][3]);
          o[1] = make_float4(acc[it][i][4], acc[it][i][5], acc[it][i][6], acc[it][i][7]);
        }
        __syncthreads();
        if (slot == 0) {
          for (int s = 1; s < slots; ++s) {
            const float4* o = reinterpret_cast<const float4*>(xslot + ((int64_t)(s - 1) * T + tl) * 8);
            const float4 a = o[0], b = o[1];
            acc[it][i][0] += a.x; acc[it][i][1] += a.y; acc[it][i][2] += a.z; acc[it][i][3] += a.w;
            acc[it][i][4] += b.x; acc[it][i][5] += b.y; acc[it][i][6] += b.z; acc[it][i][7] += b.w;
          }
        }
      }
      if (slot == 0 && act[it]) {
        float4* o = reinterpret_cast<float4*>(pr + i * SEG + 8 * cidx[it]);
        o[0] = make_float4(acc[it][i][0], acc[it][i][1], acc[it][i][2], acc[it][i][3]);
        o[1] = make_float4(acc[it][i][4], acc[it][i][5], acc[it][i][6], acc[it][i][7]);
      }
    }
  }
}

// dw[c] = sum_p partials[p, c] in a fixed order: 32 columns x 8 row lanes per workgroup, each lane sums rows
// p = lane, lane+8, ... and the 8 lane sums are added in lane order.  The kernel is one round trip to memory long, so
// a lane asks for all of its rows at once (32 loads in flight cover the 256 partial rows of the fast backward; rows
// past the end lie beyond the buffer resource and read zeros).
__global__ void __launch_bounds__(256)
k_colsum(const float* __restrict__ partials, int64_t P, int64_t H, void* __restrict__ dw, bool wf32) {
  __shared__ float part[8][33];
  constexpr int BATCH = 32;
  const int cx = threadIdx.x & 31, lane = threadIdx.x >> 5;
  const int64_t c = (int64_t)blockIdx.x * 32 + cx;
  float s = 0.f;
  for (int64_t p0 = 0; p0 < P; p0 += 8 * BATCH) {
    // rows p0 .. of the partial matrix as one resource (a batch spans at most 256 rows of at most 256 KB)
    const int64_t rows = P - p0 < 8 * BATCH ? P - p0 : 8 * BATCH;
    const BufferRsrc rs = make_rsrc(partials + p0 * H, (uint32_t)(rows * H * 4));
    const uint32_t off = c < H ? (uint32_t)((lane * H + c) * 4) : NOWHERE;
    float t[BATCH];
#pragma unroll
    for (int i = 0; i < BATCH; ++i) t[i] = __uint_as_float(load_b32(rs, off + (uint32_t)i * (uint32_t)(8 * H * 4)));
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int i = 0; i < BATCH; i += 4) { s0 += t[i]; s1 += t[i + 1]; s2 += t[i + 2]; s3 += t[i + 3]; }
    s += (s0 + s1) + (s2 + s3);
  }
  part[lane][cx] = s;
  __syncthreads();
  if (lane == 0 && c < H) {
    float tot = 0.f;
#pragma unroll
    for (int l = 0; l < 8; ++l) tot += part[l][cx];
    if (wf32) static_cast<float*>(dw)[c] = tot;
    else static_cast<uint16_t*>(dw)[c] = f_to_bf(tot);
  }
}

// Row-slot geometry of the fused norm kernels: T threads per row, ITERS chunks per thread and segment.
struct NormGeom {
  int T, iters, iters_t;   // iters_t = the template value (1, 2 or 4) that covers `iters`
};
static inline int norm_geom(int cps, NormGeom* n) {
  // one chunk per thread and segment whenever a workgroup can span the row: light threads, high occupancy
  int T = cps <= 1024 ? ((cps + 63) / 64) * 64 : 1024;
  int iters = (cps + T - 1) / T;
  if (iters > 4) return fail(HYC_ENOTSUP, "row too long for the fused RMSNorm kernels (%d chunks per segment)", cps);
  n->T = T;
  n->iters = iters;
  n->iters_t = iters <= 1 ? 1 : (iters <= 2 ? 2 : 4);
  return HYC_OK;
}

constexpr int BWD_FAST_SLOTS_MAX = 4;      // row slots per workgroup of the fast backward kernel, at most
constexpr int BWD_FAST_THREADS_MAX = 1024; // ... and its thread bound (the static LDS queue is sized by it)
constexpr int BWD_SLOTS_SMALL = 1;         // row slots per workgroup of the generic backward kernel on narrow rows
// backward launch shape: slots per workgroup and rows per workgroup
struct BwdShape {
  int slots, threads, rpb;
  int64_t P;
  int fast_slots;      // fast path: row slots per workgroup and workgroups (= partial rows)
  int fast_T;          //   threads per row slot (two threads share a packed word of 2-bit codes)
  bool fast_ok;
  bool fast_long;      //   rows so long that the queue holds two stages, not three
  int64_t fast_P;
};
static inline BwdShape bwd_shape(int64_t M, int bits, int cps, const NormGeom& n) {
  BwdShape b;
  const int parts = bits == 2 ? 2 : 1;
  b.fast_T = ((parts * cps + 63) / 64) * 64;
  b.fast_ok = n.iters == 1 && bits != 1 && b.fast_T <= 1024;
  b.fast_long = false;
  if (b.fast_ok) {
    // LDS of the fast kernel: the dy queue and the row sums (static, sized by the kernel's thread bound) and the
    // weight row (dynamic); 160 KB per workgroup on gfx950
    int fs0 = 1024 / b.fast_T;
    if (fs0 > BWD_FAST_SLOTS_MAX) fs0 = BWD_FAST_SLOTS_MAX;
    const int64_t maxt = fs0 * b.fast_T <= 256 ? 256 : BWD_FAST_THREADS_MAX, nseg = bits == 8 ? 1 : 2;
    if (fs0 * b.fast_T > BWD_FAST_THREADS_MAX) b.fast_ok = false;
    const int64_t H = (int64_t)cps * 64 / bits;
    const int64_t lds = RING_D * maxt * nseg * 16 + 1024 + H * 4;
    // (a queue of two stages where three do not fit: one row slot of 1024 threads)
    b.fast_long = b.fast_ok && lds > 160 * 1024 && maxt == 1024 && 2 * maxt * nseg * 16 + 1024 + H * 4 <= 160 * 1024;
    b.fast_ok = b.fast_ok && (lds <= 160 * 1024 || b.fast_long);
  }
  b.slots = n.T <= 256 ? BWD_SLOTS_SMALL : 1;
  b.threads = b.slots * n.T;
  // about a thousand row slots in flight; each walks at least four rows so the partial rows stay few
  int64_t rpb = (M * b.slots + 1023) / 1024;
  if (rpb < 4 * b.slots) rpb = 4 * b.slots;
  rpb = ((rpb + b.slots - 1) / b.slots) * b.slots;
  b.rpb = (int)rpb;
  b.P = M > 0 ? (M + rpb - 1) / rpb : 0;
  // fast path: up to 1024 threads per workgroup, one workgroup per CU slot; every slot walks at least two rows
  const int ft = b.fast_ok ? b.fast_T : 1024;
  int fs = 1024 / ft;
  if (fs < 1) fs = 1;
  if (fs > BWD_FAST_SLOTS_MAX) fs = BWD_FAST_SLOTS_MAX;
  int64_t fp = 256 * (int64_t)(1024 / (fs * ft) > 0 ? 1024 / (fs * ft) : 1);
  const int64_t need = (M + 2 * fs - 1) / (2 * fs);
  if (fp > need) fp = need;
  if (fp < 1) fp = 1;
  b.fast_slots = fs;
  b.fast_P = M > 0 ? fp : 0;
  return b;
}

}  // namespace hyc

using namespace hyc;

#define HYC_BITS_ITERS(BITS_, ITERS_, ...)                                                  \
  do {                                                                                      \
    switch ((BITS_) * 10 + (ITERS_)) {                                                      \
      HYC_CASE_(1, 1, __VA_ARGS__) HYC_CASE_(1, 2, __VA_ARGS__) HYC_CASE_(1, 4, __VA_ARGS__)  \
      HYC_CASE_(2, 1, __VA_ARGS__) HYC_CASE_(2, 2, __VA_ARGS__) HYC_CASE_(2, 4, __VA_ARGS__)  \
      HYC_CASE_(4, 1, __VA_ARGS__) HYC_CASE_(4, 2, __VA_ARGS__) HYC_CASE_(4, 4, __VA_ARGS__)  \
      HYC_CASE_(8, 1, __VA_ARGS__) HYC_CASE_(8, 2, __VA_ARGS__) HYC_CASE_(8, 4, __VA_ARGS__)  \
      default: return fail(HYC_ENOTSUP, "unsupported bits/iters combination (bits=%d)", (BITS_)); \
    }                                                                                       \
  } while (0)
#define HYC_CASE_(B_, I_, ...) \
  case (B_) * 10 + (I_): { constexpr int B = B_, IT = I_; __VA_ARGS__; } break;

extern "C" {

int64_t hyc_rmsnorm_bwd_partials(int64_t M, int64_t H) {
  // the partial count depends on the bit width only through the slot count; report the largest over all widths
  if (M <= 0 || H <= 0) return 0;
  int64_t best = 0;
  for (int bits = 1; bits <= 8; bits *= 2) {
    if (H % (64 / bits) != 0) continue;
    NormGeom n;
    if (norm_geom((int)(H * bits / 64), &n)) continue;
    const BwdShape b = bwd_shape(M, bits, (int)(H * bits / 64), n);
    if (b.P > best) best = b.P;
    if (b.fast_P > best) best = b.fast_P;
  }
  return best;
}

int64_t hyc_rmsnorm_bwd_partial_rows(int64_t M, int64_t H, const hyc_desc* d) {
  if (!d || M <= 0 || H <= 0) return 0;
  RowGeom g;
  NormGeom n;
  if (row_geom(H, d->bits, &g) || norm_geom(g.cps, &n)) return 0;
  const BwdShape b = bwd_shape(M, d->bits, g.cps, n);
  return ((d->mode == HYC_MODE_CHANNEL && b.fast_ok) || (d->mode == HYC_MODE_DENSE && d->bits == 4 && b.fast_ok && !b.fast_long)) ? b.fast_P : b.P;
}

static int norm_fwd_impl(const void* x, const void* w, const void* bias, int32_t w_dtype, float eps, int64_t M, int64_t H,
                         const hyc_desc* d, void* y, float* mean, float* rstd, void* stored, void* vals, void* scales,
                         int32_t* row_counts, void* stream, bool ln) {
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
  NormGeom n;
  if ((rc = norm_geom(g.cps, &n))) return rc;
  if (M == 0) return HYC_OK;
  if (!x || !w || !y || !rstd || !stored || (ln && !mean)) return fail(HYC_EFAULT, "hyc_rmsnorm_fwd_compress: null buffer");
  if (ln && n.iters_t != 1)
    return fail(HYC_ENOTSUP, "hyc_layernorm_fwd_compress: rows of at most 1024 chunks per segment (H*bits/64 <= 1024)");
  if (ln && bias && !aligned16(bias)) return fail(HYC_EINVAL, "hyc_layernorm_fwd_compress: bias must be 16-byte aligned");
  if (d->mode == HYC_MODE_CHANNEL && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_rmsnorm_fwd_compress: null vals/scales");
  if (!aligned16(x) || !aligned16(y) || !aligned16(w) || !aligned8(stored))
    return fail(HYC_EINVAL, "hyc_rmsnorm_fwd_compress: x, y, w must be 16-byte and stored 8-byte aligned");
  const bool wf32 = w_dtype == HYC_DTYPE_F32;
  // workgroups: about four rows each (measured: 1024 workgroups at 4096 rows, 16 384 at 65 536), at least one round
  // of the chip, and two per CU when a row takes more than eight waves
  int64_t cap = n.T >= 512 ? 512 : (M / 4 < 1024 ? 1024 : (M / 4 > 16384 ? 16384 : M / 4));
  int grid = (int)(M < cap ? M : cap);
  hipStream_t st = begin_launch(stream);
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  // fast path: every lane owns one chunk per segment, group width known at compile time
  if (d->mode == HYC_MODE_CHANNEL && n.iters == 1 && (lpg == 8 || lpg == 16) && d->bits != 1) {
    uint16_t* yp = static_cast<uint16_t*>(y);
    uint8_t* stp = static_cast<uint8_t*>(stored);
    uint16_t* vp = static_cast<uint16_t*>(vals);
    uint16_t* scp = static_cast<uint16_t*>(scales);
#define HYC_FWD_FAST_R(B_, L_, W_, MT_, R_)                                                                        \
  do {                                                                                                             \
    const size_t qb_ = (size_t)fwd_queue_depth(MT_, Q<B_>::NSEG) * n.T * Q<B_>::NSEG * 16;                         \
    if (ln)                                                                                                        \
      hipLaunchKernelGGL((k_layernorm_fwd_fast<B_, L_, W_, MT_, R_>), dim3(grid), dim3(n.T), qb_, st, xp, w, bias, eps, M, H, \
                         g.cps, ca, yp, mean, rstd, stp, vp, scp);                                                 \
    else                                                                                                           \
      hipLaunchKernelGGL((k_rmsnorm_fwd_fast<B_, L_, W_, MT_, R_>), dim3(grid), dim3(n.T), qb_, st, xp, w, eps, M, H, \
                         g.cps, ca, yp, rstd, stp, vp, scp);                                                       \
  } while (0)
#define HYC_FWD_FAST(B_, L_, W_, MT_)                                                                              \
  do { if (ca.absmax) HYC_FWD_FAST_R(B_, L_, W_, MT_, SCALE_ABSMAX); else HYC_FWD_FAST_R(B_, L_, W_, MT_, SCALE_RANGE); } while (0)
#define HYC_FWD_FAST_W(B_, L_)                                                        \
  do {                                                                                \
    if (n.T <= 256) { if (wf32) HYC_FWD_FAST(B_, L_, true, 256); else HYC_FWD_FAST(B_, L_, false, 256); }  \
    else { if (wf32) HYC_FWD_FAST(B_, L_, true, 1024); else HYC_FWD_FAST(B_, L_, false, 1024); }           \
  } while (0)
    switch (d->bits * 100 + lpg) {
      case 208: HYC_FWD_FAST_W(2, 8); break;
      case 216: HYC_FWD_FAST_W(2, 16); break;
      case 408: HYC_FWD_FAST_W(4, 8); break;
      case 416: HYC_FWD_FAST_W(4, 16); break;
      case 808: HYC_FWD_FAST_W(8, 8); break;
      default: HYC_FWD_FAST_W(8, 16); break;
    }
#undef HYC_FWD_FAST_W
#undef HYC_FWD_FAST
#undef HYC_FWD_FAST_R
    return check_launch(ln ? "hyc_layernorm_fwd_compress" : "hyc_rmsnorm_fwd_compress");
  }
  // the general kernels keep the next row in registers, not in a queue: one row per workgroup is their best grid for
  // rows of up to 256 chunks (threshold scheme, 4096 x 4096: 18.9 -> 17.0 us, 16 384 rows: 57.8 -> 49.9 us)
  if (n.T < 512) grid = (int)(M < (int64_t)1 << 30 ? M : (int64_t)1 << 30);
#define HYC_FWD_K(KERNEL_)                                                                                         \
  hipLaunchKernelGGL(KERNEL_, dim3(grid), dim3(n.T), 0, st, xp, w, bias, wf32, eps, M, H, g.cps,                   \
                     ca, lpg, ta, perchan, static_cast<uint16_t*>(y), mean, rstd, static_cast<uint8_t*>(stored),   \
                     static_cast<uint16_t*>(vals), static_cast<uint16_t*>(scales), row_counts)
#define HYC_FWD(MODE_, MT_) HYC_FWD_K((k_rmsnorm_fwd<B, IT, MT_, MODE_>))
#define HYC_FWD_LN(B_, MODE_)                                                                                      \
  do {                                                                                                             \
    if (n.T <= 256) HYC_FWD_K((k_rmsnorm_fwd<B_, 1, 256, MODE_, true>));                                           \
    else HYC_FWD_K((k_rmsnorm_fwd<B_, 1, 1024, MODE_, true>));                                                     \
  } while (0)
  if (ln) {
#define HYC_FWD_LN_BITS(MODE_)                                  \
  switch (d->bits) {                                            \
    case 1: HYC_FWD_LN(1, MODE_); break;                        \
    case 2: HYC_FWD_LN(2, MODE_); break;                        \
    case 4: HYC_FWD_LN(4, MODE_); break;                        \
    default: HYC_FWD_LN(8, MODE_); break;                       \
  }
    if (d->mode == HYC_MODE_CHANNEL) { HYC_FWD_LN_BITS(0) } else { HYC_FWD_LN_BITS(1) }
#undef HYC_FWD_LN_BITS
    return check_launch("hyc_layernorm_fwd_compress");
  }
  if (d->mode == HYC_MODE_CHANNEL) {
    HYC_BITS_ITERS(d->bits, n.iters_t, if (n.T <= 256) HYC_FWD(0, 256); else HYC_FWD(0, 1024));
  } else {
    HYC_BITS_ITERS(d->bits, n.iters_t, if (n.T <= 256) HYC_FWD(1, 256); else HYC_FWD(1, 1024));
  }
#undef HYC_FWD
#undef HYC_FWD_LN
#undef HYC_FWD_K
  return check_launch("hyc_rmsnorm_fwd_compress");
}

int hyc_rmsnorm_fwd_compress(const void* x, const void* w, int32_t w_dtype, float eps, int64_t M, int64_t H,
                             const hyc_desc* d, void* y, float* rstd, void* stored, void* vals, void* scales,
                             int32_t* row_counts, void* stream) {
  return norm_fwd_impl(x, w, nullptr, w_dtype, eps, M, H, d, y, nullptr, rstd, stored, vals, scales, row_counts, stream, false);
}

int hyc_layernorm_fwd_compress(const void* x, const void* w, const void* bias, int32_t w_dtype, float eps, int64_t M,
                               int64_t H, const hyc_desc* d, void* y, float* mean, float* rstd, void* stored, void* vals,
                               void* scales, int32_t* row_counts, void* stream) {
  return norm_fwd_impl(x, w, bias, w_dtype, eps, M, H, d, y, mean, rstd, stored, vals, scales, row_counts, stream, true);
}

static int norm_bwd_impl(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                         int32_t w_dtype, const float* rstd, const float* mean, int64_t M, int64_t H, const hyc_desc* d,
                         int32_t c2_quirk, void* dx, float* dw_partials, void* dw, void* stream) {
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
  NormGeom n;
  if ((rc = norm_geom(g.cps, &n))) return rc;
  hipStream_t st = begin_launch(stream);
  const bool wf32 = w_dtype == HYC_DTYPE_F32;
  const BwdShape b = bwd_shape(M, d->bits, g.cps, n);
  // the dense source takes the fast kernel through the chunk mapping of 4-bit codes (two half rows per thread)
  const bool dense_fast = d->mode == HYC_MODE_DENSE && d->bits == 4 && b.fast_ok && !b.fast_long;
  const bool fast = (d->mode == HYC_MODE_CHANNEL && b.fast_ok) || dense_fast;
  const int64_t used_P = fast ? b.fast_P : b.P;
  if (M > 0) {
    if (!dy || !stored || !w || !rstd || !dx || !dw_partials) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null buffer");
    if (d->mode == HYC_MODE_CHANNEL && (!scales || (d->k > 0 && !vals))) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd: null vals/scales");
    if (!aligned16(dy) || !aligned16(dx) || !aligned16(w) || !aligned16(dw_partials) || !aligned8(stored) ||
        (d->mode == HYC_MODE_DENSE && !aligned16(stored)))
      return fail(HYC_EINVAL, "hyc_rmsnorm_bwd: dy, dx, w, dw_partials must be 16-byte aligned, stored 8-byte (16 when dense)");
    const uint16_t* gp = static_cast<const uint16_t*>(dy);
    const size_t lds = b.slots > 1 ? (size_t)(b.slots - 1) * n.T * 8 * sizeof(float) : 0;
    if (fast) {
      const int fthreads = b.fast_slots * b.fast_T;
      const size_t flds = (size_t)H * sizeof(float);
      const int64_t fstride = b.fast_P * b.fast_slots;
      const int fsteps = (int)((M + fstride - 1) / fstride);
#define HYC_BWD_FAST(B_, W_, Q_, MT_)                                                                              \
  hipLaunchKernelGGL((k_rmsnorm_bwd_fast<B_, W_, Q_, MT_>), dim3((unsigned)b.fast_P), dim3(fthreads), flds, st, gp,  \
                     static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                     \
                     static_cast<const uint16_t*>(scales), w, rstd, mean, M, H, b.fast_T, g.cps, b.fast_slots, fsteps, ca, \
                     static_cast<uint16_t*>(dx), dw_partials)
#define HYC_BWD_FAST_WQ(B_)                                                                   \
  do {                                                                                        \
    const int key_ = (wf32 ? 4 : 0) + (c2_quirk ? 2 : 0) + (fthreads <= 256 ? 0 : 1);        \
    switch (key_) {                                                                           \
      case 0: HYC_BWD_FAST(B_, false, false, 256); break;                                     \
      case 1: HYC_BWD_FAST(B_, false, false, BWD_FAST_THREADS_MAX); break;                                    \
      case 2: HYC_BWD_FAST(B_, false, true, 256); break;                                      \
      case 3: HYC_BWD_FAST(B_, false, true, BWD_FAST_THREADS_MAX); break;                                     \
      case 4: HYC_BWD_FAST(B_, true, false, 256); break;                                      \
      case 5: HYC_BWD_FAST(B_, true, false, BWD_FAST_THREADS_MAX); break;                                     \
      case 6: HYC_BWD_FAST(B_, true, true, 256); break;                                       \
      default: HYC_BWD_FAST(B_, true, true, BWD_FAST_THREADS_MAX); break;                                     \
    }                                                                                         \
  } while (0)
      if (dense_fast) {
#define HYC_BWD_DENSE(W_, Q_, MT_)                                                                                 \
  hipLaunchKernelGGL((k_rmsnorm_bwd_fast<4, W_, Q_, MT_, true>), dim3((unsigned)b.fast_P), dim3(fthreads), flds, st, gp, \
                     static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                     \
                     static_cast<const uint16_t*>(scales), w, rstd, mean, M, H, b.fast_T, g.cps, b.fast_slots, fsteps, ca, \
                     static_cast<uint16_t*>(dx), dw_partials)
        switch ((wf32 ? 4 : 0) + (c2_quirk ? 2 : 0) + (fthreads <= 256 ? 0 : 1)) {
          case 0: HYC_BWD_DENSE(false, false, 256); break;
          case 1: HYC_BWD_DENSE(false, false, BWD_FAST_THREADS_MAX); break;
          case 2: HYC_BWD_DENSE(false, true, 256); break;
          case 3: HYC_BWD_DENSE(false, true, BWD_FAST_THREADS_MAX); break;
          case 4: HYC_BWD_DENSE(true, false, 256); break;
          case 5: HYC_BWD_DENSE(true, false, BWD_FAST_THREADS_MAX); break;
          case 6: HYC_BWD_DENSE(true, true, 256); break;
          default: HYC_BWD_DENSE(true, true, BWD_FAST_THREADS_MAX); break;
        }
#undef HYC_BWD_DENSE
      }
      else if (b.fast_long) {
#define HYC_BWD_LONG(B_, W_, Q_)                                                                                   \
  hipLaunchKernelGGL((k_rmsnorm_bwd_fast_long<B_, W_, Q_>), dim3((unsigned)b.fast_P), dim3(fthreads), flds, st, gp, \
                     static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                     \
                     static_cast<const uint16_t*>(scales), w, rstd, mean, M, H, b.fast_T, g.cps, b.fast_slots, fsteps, ca, \
                     static_cast<uint16_t*>(dx), dw_partials)
#define HYC_BWD_LONG_WQ(B_)                                                                                        \
  do {                                                                                                             \
    if (wf32) { if (c2_quirk) HYC_BWD_LONG(B_, true, true); else HYC_BWD_LONG(B_, true, false); }                  \
    else { if (c2_quirk) HYC_BWD_LONG(B_, false, true); else HYC_BWD_LONG(B_, false, false); }                     \
  } while (0)
        if (d->bits == 2) HYC_BWD_LONG_WQ(2); else if (d->bits == 4) HYC_BWD_LONG_WQ(4); else HYC_BWD_LONG_WQ(8);
#undef HYC_BWD_LONG_WQ
#undef HYC_BWD_LONG
      }
      else if (d->bits == 2) HYC_BWD_FAST_WQ(2);
      else if (d->bits == 4) HYC_BWD_FAST_WQ(4);
      else HYC_BWD_FAST_WQ(8);
#undef HYC_BWD_FAST_WQ
#undef HYC_BWD_FAST
      if ((rc = check_launch("hyc_rmsnorm_bwd"))) return rc;
    } else {
#define HYC_BWD(SRC_)                                                                                             \
  if (IT == 1 && b.threads <= 256)                                                                                \
    hipLaunchKernelGGL((k_rmsnorm_bwd<B, IT, (IT == 1 ? 256 : 1024), SRC_>), dim3((unsigned)b.P), dim3(b.threads), lds, st, gp, \
                       static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                   \
                       static_cast<const uint16_t*>(scales), w, wf32, rstd, mean, M, H, g.cps, n.T, b.slots, b.rpb, ca, \
                       c2_quirk != 0, static_cast<uint16_t*>(dx), dw_partials);                                   \
  else if (IT == 1 && b.threads <= 512)                                                                           \
    hipLaunchKernelGGL((k_rmsnorm_bwd<B, IT, (IT == 1 ? 512 : 1024), SRC_>), dim3((unsigned)b.P), dim3(b.threads), lds, st, gp, \
                       static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                   \
                       static_cast<const uint16_t*>(scales), w, wf32, rstd, mean, M, H, g.cps, n.T, b.slots, b.rpb, ca, \
                       c2_quirk != 0, static_cast<uint16_t*>(dx), dw_partials);                                   \
  else                                                                                                            \
  hipLaunchKernelGGL((k_rmsnorm_bwd<B, IT, 1024, SRC_>), dim3((unsigned)b.P), dim3(b.threads), lds, st, gp,       \
                     static_cast<const uint8_t*>(stored), static_cast<const uint16_t*>(vals),                     \
                     static_cast<const uint16_t*>(scales), w, wf32, rstd, mean, M, H, g.cps, n.T, b.slots, b.rpb, ca, \
                     c2_quirk != 0, static_cast<uint16_t*>(dx), dw_partials)
    if (d->mode == HYC_MODE_CHANNEL) HYC_BITS_ITERS(d->bits, n.iters_t, HYC_BWD(0));
    else HYC_BITS_ITERS(d->bits, n.iters_t, HYC_BWD(2));
#undef HYC_BWD
    if ((rc = check_launch("hyc_rmsnorm_bwd"))) return rc;
    }
  }
  if (!dw) return HYC_OK;                        // the caller adds up the partial rows itself
  hipLaunchKernelGGL(k_colsum, dim3((unsigned)((H + 31) / 32)), dim3(256), 0, st, dw_partials, used_P, H, dw, wf32);
  return check_launch("hyc_rmsnorm_bwd (dw)");
}

int hyc_rmsnorm_bwd(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                    int32_t w_dtype, const float* rstd, int64_t M, int64_t H, const hyc_desc* d, int32_t c2_quirk,
                    void* dx, float* dw_partials, void* dw, void* stream) {
  return norm_bwd_impl(dy, stored, vals, scales, w, w_dtype, rstd, nullptr, M, H, d, c2_quirk, dx, dw_partials, dw, stream);
}

// ---- the backward for callers that cannot allocate -------------------------------------------------------------
// The fp32 partial rows of dw live in a file-scope device array instead of a caller buffer.  In host code the
// array's name is only a handle: the address the kernels need is asked from the runtime once per device (each
// device holds its own copy of the array) and kept.
static __device__ __align__(256) float scratch[HYC_RMSNORM_BWD_STATIC_MAX_FLOATS];

static int static_scratch(float** out, hipStream_t stream) {
  static std::atomic<float*> per_device[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(HYC_ELAUNCH, "hyc_rmsnorm_bwd_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= 64) return fail(HYC_ENOTSUP, "hyc_rmsnorm_bwd_static: device ordinal %d (0..63 are covered)", dev);
  float* p = per_device[dev].load(std::memory_order_acquire);
  if (!p) {
    // asking the runtime for the address is not a stream operation: under a capture it could fail or end the capture,
    // so a first call that arrives there is refused instead (any earlier call on this device, M = 0 included, avoids it)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    e = hipStreamIsCapturing(stream, &cap);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(HYC_ELAUNCH, "hyc_rmsnorm_bwd_static: hipStreamIsCapturing: %s", hipGetErrorString(e));
    }
    if (cap != hipStreamCaptureStatusNone)
      return fail(HYC_EINVAL, "hyc_rmsnorm_bwd_static: the first call on a device resolves the workspace address and must be "
                  "made outside a stream capture (a call with M = 0 is enough)");
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sym) {
      (void)hipGetLastError();
      return fail(HYC_ELAUNCH, "hyc_rmsnorm_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    }
    p = static_cast<float*>(sym);
    per_device[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return HYC_OK;
}

int hyc_rmsnorm_bwd_static(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                           int32_t w_dtype, const float* rstd, int64_t M, int64_t H, const hyc_desc* d, int32_t c2_quirk,
                           void* dx, void* dw, void* stream) {
  if (!d) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd_static: null descriptor");
  if (M > 0 && !dw) return fail(HYC_EFAULT, "hyc_rmsnorm_bwd_static: dw is required (the partial rows are not the caller's)");
  const int64_t rows = hyc_rmsnorm_bwd_partial_rows(M, H, d);
  if (rows * H > (int64_t)HYC_RMSNORM_BWD_STATIC_MAX_FLOATS)
    return fail(HYC_EINVAL, "hyc_rmsnorm_bwd_static: %lld partial rows of %lld floats exceed the static workspace of %lld floats; "
                "use hyc_rmsnorm_bwd with a caller workspace", (long long)rows, (long long)H,
                (long long)HYC_RMSNORM_BWD_STATIC_MAX_FLOATS);
  float* partials = nullptr;
  const int rc = static_scratch(&partials, static_cast<hipStream_t>(stream));
  if (rc) return rc;
  if (M == 0) return HYC_OK;                     // nothing to do: the call has resolved the workspace address
  return norm_bwd_impl(dy, stored, vals, scales, w, w_dtype, rstd, nullptr, M, H, d, c2_quirk, dx, partials, dw, stream);
}

int hyc_layernorm_bwd(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                      int32_t w_dtype, const float* mean, const float* rstd, int64_t M, int64_t H, const hyc_desc* d,
                      void* dx, float* dw_partials, void* dw, void* stream) {
  if (M > 0 && !mean) return fail(HYC_EFAULT, "hyc_layernorm_bwd: null mean");
  return norm_bwd_impl(dy, stored, vals, scales, w, w_dtype, rstd, mean, M, H, d, 1, dx, dw_partials, dw, stream);
}

}  // extern "C"
