// Rotary position embedding fused with the layout change attention needs (reference: apply_rotary_pos_emb and the
// `.view(b, s, nh, hd).transpose(1, 2)` around it, models/modeling_llama.py:236-260 and :423-425).  The projections
// produce [B, S, nh, hd]; the batched attention GEMMs want [B, nh, S, hd] contiguous; the framework does this with
// five elementwise kernels per tensor plus a layout copy inside the GEMM.  Here one streaming pass reads x once and
// writes the rotated tensor in the head-major layout and, when asked, in the row-major layout too (the rows are
// what gets compressed).  The backward is the transposed rotation from head-major gradients to row-major.
//   y[i]     = x[i]     * cos[i]     - x[i+h] * sin[i]          (i < h = hd/2)
//   y[i+h]   = x[i+h]   * cos[i+h]   + x[i]   * sin[i+h]
//   dx[i]    = g[i]     * cos[i]     + g[i+h] * sin[i+h]
//   dx[i+h]  = g[i+h]   * cos[i+h]   - g[i]   * sin[i]
// fp32 arithmetic, one rounding to bf16 (the reference rounds each of its three elementwise steps).
#include "abi_util.hpp"

namespace hyc {

// division by a launch constant: a shift when it is a power of two (every LLaMA shape), a real division otherwise
struct Divisor {
  uint32_t d;
  int shift;     // >= 0: d == 1 << shift
  __device__ __forceinline__ uint32_t div(uint32_t x) const { return shift >= 0 ? x >> shift : x / d; }
};
static Divisor make_divisor(int64_t d) {
  Divisor r{(uint32_t)d, -1};
  for (int sft = 0; sft < 31; ++sft)
    if (((int64_t)1 << sft) == d) r.shift = sft;
  return r;
}

// An item is 8 channels of the low half and the matching 8 of the high half of one (b, s, head); fewer than 2^31 items.
// TO_HEADS: in = rows layout, out_heads (and optionally out_rows); else in = heads layout, out = rows layout.
template <bool TO_HEADS, bool ROTATE>
__global__ void __launch_bounds__(256)
k_rope(const uint16_t* __restrict__ in, const uint16_t* __restrict__ cosv, const uint16_t* __restrict__ sinv,
       uint32_t items, Divisor per_head, Divisor heads, Divisor seq, int hd, int64_t in_pitch,
       uint16_t* __restrict__ out_heads, uint16_t* __restrict__ out_rows) {
  const int half = hd / 2;
  const uint32_t step = gridDim.x * 256u;
  for (uint32_t t = blockIdx.x * 256u + threadIdx.x; t < items; t += step) {
    const uint32_t bsh = per_head.div(t), sub = t - bsh * per_head.d;
    const uint32_t bs = heads.div(bsh), h = bsh - bs * heads.d;
    const uint32_t b = seq.div(bs), s = bs - b * seq.d;
    const int64_t rows_off = (int64_t)bsh * hd + 8 * sub;                                              // [b, s, h, d]
    const int64_t heads_off = (((int64_t)b * heads.d + h) * seq.d + s) * hd + 8 * sub;               // [b, h, s, d]
    // a row-major input may be a column slice of a wider matrix: its tokens are in_pitch elements apart
    const int64_t in_off = TO_HEADS ? (int64_t)bs * in_pitch + (int64_t)h * hd + 8 * sub : heads_off;
    float lo[8], hi[8];
    const uint4 rlo = *reinterpret_cast<const uint4*>(in + in_off);
    const uint4 rhi = *reinterpret_cast<const uint4*>(in + in_off + half);
    uint4 wlo = rlo, whi = rhi;
    if (ROTATE) {
      float cl[8], ch[8], sl[8], sh[8];
      unpack8(rlo, lo);
      unpack8(rhi, hi);
      const int64_t tab = (int64_t)s * hd + 8 * sub;
      unpack8(*reinterpret_cast<const uint4*>(cosv + tab), cl);
      unpack8(*reinterpret_cast<const uint4*>(cosv + tab + half), ch);
      unpack8(*reinterpret_cast<const uint4*>(sinv + tab), sl);
      unpack8(*reinterpret_cast<const uint4*>(sinv + tab + half), sh);
      float ol[8], oh[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (TO_HEADS) {
          ol[j] = __builtin_fmaf(lo[j], cl[j], -(hi[j] * sl[j]));
          oh[j] = __builtin_fmaf(hi[j], ch[j], lo[j] * sh[j]);
        } else {
          ol[j] = __builtin_fmaf(lo[j], cl[j], hi[j] * sh[j]);
          oh[j] = __builtin_fmaf(hi[j], ch[j], -(lo[j] * sl[j]));
        }
      }
      wlo = pack8(ol);
      whi = pack8(oh);
    }
    if (TO_HEADS) {
      *reinterpret_cast<uint4*>(out_heads + heads_off) = wlo;
      *reinterpret_cast<uint4*>(out_heads + heads_off + half) = whi;
      if (out_rows) {
        *reinterpret_cast<uint4*>(out_rows + rows_off) = wlo;
        *reinterpret_cast<uint4*>(out_rows + rows_off + half) = whi;
      }
    } else {
      *reinterpret_cast<uint4*>(out_rows + rows_off) = wlo;
      *reinterpret_cast<uint4*>(out_rows + rows_off + half) = whi;
    }
  }
}

static int rope_args(const char* who, int64_t B, int64_t S, int64_t nh, int64_t hd) {
  if (B < 0 || S < 0 || nh <= 0 || hd <= 0 || hd % 16 != 0 || hd > 1024 || nh > 65536)
    return fail(HYC_EINVAL, "%s: B=%lld S=%lld heads=%lld head_dim=%lld (head_dim must be a multiple of 16, at most 1024)",
                who, (long long)B, (long long)S, (long long)nh, (long long)hd);
  if (S > 0 && B * S * nh > (((int64_t)1 << 31) - 1) / (hd / 16))      // 32-bit item counter with room for its stride
    return fail(HYC_EINVAL, "%s: B*S*heads*head_dim/16 must stay below 2^31", who);
  return HYC_OK;
}

static unsigned rope_grid(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}

}  // namespace hyc

using namespace hyc;

extern "C" {

int hyc_rope_to_heads(const void* x, int64_t x_pitch, const void* cosv, const void* sinv, int64_t B, int64_t S,
                      int64_t heads, int64_t head_dim, void* out_heads, void* out_rows, void* stream) {
  int rc = rope_args("hyc_rope_to_heads", B, S, heads, head_dim);
  if (rc) return rc;
  if (x_pitch < heads * head_dim || x_pitch % 8 != 0)
    return fail(HYC_EINVAL, "hyc_rope_to_heads: token pitch %lld (at least heads*head_dim, a multiple of 8)", (long long)x_pitch);
  if (B == 0 || S == 0) return HYC_OK;
  if (!x || !out_heads || ((cosv == nullptr) != (sinv == nullptr))) return fail(HYC_EFAULT, "hyc_rope_to_heads: null buffer");
  if (!aligned16(x) || !aligned16(out_heads) || !aligned16(out_rows) || !aligned16(cosv) || !aligned16(sinv))
    return fail(HYC_EINVAL, "hyc_rope_to_heads: buffers must be 16-byte aligned");
  const int64_t items = B * S * heads * (head_dim / 16);
  const dim3 grid(rope_grid(items));
  hipStream_t st = begin_launch(stream);
  if (cosv)
    hipLaunchKernelGGL((k_rope<true, true>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(x),
                       static_cast<const uint16_t*>(cosv), static_cast<const uint16_t*>(sinv), (uint32_t)items,
                       make_divisor(head_dim / 16), make_divisor(heads), make_divisor(S), (int)head_dim, x_pitch,
                       static_cast<uint16_t*>(out_heads), static_cast<uint16_t*>(out_rows));
  else
    hipLaunchKernelGGL((k_rope<true, false>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(x),
                       static_cast<const uint16_t*>(nullptr), static_cast<const uint16_t*>(nullptr), (uint32_t)items,
                       make_divisor(head_dim / 16), make_divisor(heads), make_divisor(S), (int)head_dim, x_pitch,
                       static_cast<uint16_t*>(out_heads), static_cast<uint16_t*>(out_rows));
  return check_launch("hyc_rope_to_heads");
}

int hyc_rope_from_heads(const void* g, const void* cosv, const void* sinv, int64_t B, int64_t S, int64_t heads,
                        int64_t head_dim, void* out_rows, void* stream) {
  int rc = rope_args("hyc_rope_from_heads", B, S, heads, head_dim);
  if (rc) return rc;
  if (B == 0 || S == 0) return HYC_OK;
  if (!g || !out_rows || ((cosv == nullptr) != (sinv == nullptr))) return fail(HYC_EFAULT, "hyc_rope_from_heads: null buffer");
  if (!aligned16(g) || !aligned16(out_rows) || !aligned16(cosv) || !aligned16(sinv))
    return fail(HYC_EINVAL, "hyc_rope_from_heads: buffers must be 16-byte aligned");
  const int64_t items = B * S * heads * (head_dim / 16);
  const dim3 grid(rope_grid(items));
  hipStream_t st = begin_launch(stream);
  if (cosv)
    hipLaunchKernelGGL((k_rope<false, true>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(g),
                       static_cast<const uint16_t*>(cosv), static_cast<const uint16_t*>(sinv), (uint32_t)items,
                       make_divisor(head_dim / 16), make_divisor(heads), make_divisor(S), (int)head_dim, (int64_t)0,
                       static_cast<uint16_t*>(nullptr), static_cast<uint16_t*>(out_rows));
  else
    hipLaunchKernelGGL((k_rope<false, false>), grid, dim3(256), 0, st, static_cast<const uint16_t*>(g),
                       static_cast<const uint16_t*>(nullptr), static_cast<const uint16_t*>(nullptr), (uint32_t)items,
                       make_divisor(head_dim / 16), make_divisor(heads), make_divisor(S), (int)head_dim, (int64_t)0,
                       static_cast<uint16_t*>(nullptr), static_cast<uint16_t*>(out_rows));
  return check_launch("hyc_rope_from_heads");
}

}  // extern "C"
