/*
 * hyc_abi.h - C ABI of the MI355X (gfx950) hybrid activation-compression library.
 *
 * Plain pointers and sizes only; every pointer named "device" is HBM memory of the current HIP
 * device, every entry point is asynchronous on the given stream (a hipStream_t passed as void*,
 * NULL = the default stream), returns 0 on success or a negative HYC_E* code, never throws,
 * never synchronises, and never allocates device memory: outputs and workspaces belong to the
 * caller.  hyc_last_error() returns a thread-local description of the last failure.
 *
 * What each entry point stands in for (paths relative to the HyC-LoRA reference checkout):
 *   hyc_compress / hyc_decompress
 *       true_divide_outlier_suboutlier_svd_compress / _decompress,
 *       operators/compress_function.py:136-200 and :203-261
 *   hyc_ref_outlier_count / hyc_ref_outlier_fill
 *       the `.to_sparse()` of the element-threshold outliers, operators/compress_function.py:149-156
 *   hyc_channel_absmax / hyc_select_channels
 *       the calibration statistics, operators/compress_function.py:292-340 (get_statistics), for the
 *       channel-structured outlier rule
 *   hyc_kth_value
 *       torch.kthvalue(x[0].flatten().float(), k).values, the calibration quantile of
 *       operators/compress_function.py:319 (get_statistics) and :345 (get_statistics_softmax)
 *   hyc_rmsnorm_fwd_compress
 *       EfficientMemoryRMSNormFunc.forward + _rms_norm_fwd_fused, operators/efficient_rmsnorm.py:147-212, :15-60
 *   hyc_rmsnorm_bwd
 *       EfficientMemoryRMSNormFunc.backward + _rms_norm_bwd_dx_fused + _rms_norm_bwd_dwdb,
 *       operators/efficient_rmsnorm.py:215-269, :63-143
 *   hyc_rmsnorm_bwd_static
 *       no counterpart in the reference: hyc_rmsnorm_bwd for callers that cannot allocate (see its declaration)
 *   hyc_act_bwd
 *       EfficientMemorySiLUFunc.backward operators/efficient_silu.py:44-53,
 *       EfficientMemoryGELUFunc.backward operators/efficient_gelu.py:44-64,
 *       EfficientMemoryHadamardFunc.backward operators/efficient_hadamard.py:55-83
 *   hyc_softmax_fwd_compress / hyc_softmax_bwd
 *       EfficientMemorySoftmaxFunc operators/efficient_softmax.py:10-45 with
 *       true_compress_softmax / true_decompress_softmax operators/compress_function.py:264-275
 *   hyc_gradw_gemm
 *       grad_weight = grad_output^T @ decompress(x), operators/efficient_linear.py:56-67
 *   hyc_low_rank_update
 *       low_rank_extraction / low_rank_addition, operators/fused_compression.py:80-99, :184-210
 *   hyc_rope_to_heads / hyc_rope_from_heads
 *       apply_rotary_pos_emb and the head-major transposition around it, models/modeling_llama.py:236-260, :423-425
 *   hyc_dropout
 *       EfficientMemoryDropoutFunc (_seeded_dropout / _seeded_dropout_backward), operators/efficient_dropout.py:7-79
 *   hyc_nf4_dequantize / hyc_nf4_quantize
 *       F.dequantize_4bit(B, quant_state) before each frozen-base matmul, bitsandbytes_fix/_function.py:509, :540
 *       (the quantiser that wrote B is bitsandbytes' own and is not part of the reference tree)
 *
 * Compressed activation of a [M, H] bf16 matrix (M tokens, H channels), `bits` in {1,2,4,8}:
 *   stored   uint8 [M, H*bits/8]   (bits == 8: int8 [M, H], the signed code itself)
 *            byte j of a row = sum_i code[j + i*H/n] << (i*bits), n = 8/bits, code = q + 2^(bits-1),
 *            q = clamp(rint(bf16(x / scale)), -2^(bits-1), 2^(bits-1)-1)   (compress_function.py:170-197)
 *   HYC_MODE_CHANNEL   k outlier channels kept verbatim: vals bf16 [M, k] (column i = channel idx[i],
 *            idx ascending); scales bf16 [M, H/group], one per token and group of channels, formed by
 *            the descriptor's scale_rule (HYC_SCALE_*) after the outlier channels were zeroed.
 *   HYC_MODE_THRESHOLD outliers are the elements with |x - base| > threshold (CSR: row_ptr int32 [M+1],
 *            cols int32 [nnz] ascending within a row, vals bf16 [nnz]); static scale read through two
 *            strides (per-tensor 0/0, per-channel 0/1, per-token 1/0) at row (m mod S);
 *            base = bf16(L[m mod S, :] @ R) with L bf16 [S, rank], R bf16 [rank, H] (rank may be 0).
 */
#ifndef HYC_ABI_H
#define HYC_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HYC_ABI_VERSION 3

/* error codes (negative errno values) */
#define HYC_OK 0
#define HYC_EINVAL (-22)  /* bad shape, misaligned pointer, inconsistent descriptor */
#define HYC_EFAULT (-14)  /* null pointer where data is required */
#define HYC_ENOTSUP (-95) /* bits / group / H combination the kernels do not cover */
#define HYC_ELAUNCH (-5)  /* the HIP runtime refused the launch */

#define HYC_MODE_CHANNEL 0
#define HYC_MODE_THRESHOLD 1
#define HYC_MODE_DENSE 2 /* consumers only: `stored` is the already decompressed bf16 [M,H] */

/* group scale of the channel scheme, over the group's channels after the outlier channels were zeroed:
 *   HYC_SCALE_RANGE   bf16(bf16(max - min) / (2^bits - 1)), the reference's formula (compress_function.py:328-334).
 *                     There is no zero point, so a group that is not centred on 0 clips at the code bounds.
 *   HYC_SCALE_ABSMAX  bf16(bf16(2 max|x|) / (2^bits - 1)): the same formula over the interval made symmetric about 0,
 *                     [-max|x|, max|x|]; no element is reconstructed more than half a step away.  (1-bit codes: max|x|.) */
#define HYC_SCALE_RANGE 0
#define HYC_SCALE_ABSMAX 1

#define HYC_DTYPE_BF16 0
#define HYC_DTYPE_F32 1

#define HYC_ACT_SILU 0
#define HYC_ACT_GELU_TANH 1

typedef struct hyc_desc {
  int32_t mode;  /* HYC_MODE_* */
  int32_t bits;  /* 1, 2, 4, 8 */
  /* ---- HYC_MODE_CHANNEL ---- */
  int32_t group; /* channels per scale group */
  int32_t k;     /* number of outlier channels (may be 0) */
  const uint32_t* chan_plan; /* device [H/8]: bits 0-7 = outlier mask of channels 8c..8c+7,
                                bits 16-31 = number of outlier channels below 8c; from hyc_select_channels */
  /* ---- HYC_MODE_THRESHOLD ---- */
  float threshold;            /* compared as bf16: the library rounds it to bf16 (nearest even) */
  const void* scale;          /* device bf16 */
  int64_t scale_stride_token; /* element (s, c) is scale[s*stride_token + c*stride_channel] */
  int64_t scale_stride_channel;
  int64_t S;                  /* rows per batch element: row m uses sequence position m mod S */
  const void* L;              /* device bf16 [S, rank] or NULL when rank == 0 */
  const void* R;              /* device bf16 [rank, H] */
  int32_t rank;
  /* ---- HYC_MODE_CHANNEL: how the encoders form the scale of a (token, group); decoders only read scales ---- */
  int32_t scale_rule; /* HYC_SCALE_* */
  /* outliers as CSR; consumed by decompress / backward entry points, produced by hyc_ref_outlier_fill */
  const int32_t* csr_row_ptr; /* device [M+1] */
  const int32_t* csr_cols;    /* device [nnz] */
  const void* csr_vals;       /* device bf16 [nnz] */
  /* ---- HYC_MODE_CHANNEL (continued) ---- */
  const int32_t* chan_idx;    /* device [k]: the outlier channels, ascending (from hyc_select_channels); needed when k > 0 */
} hyc_desc;

int hyc_abi_version(void);
const char* hyc_last_error(void);

/* 0 when the kernels cover (H, bits, group) in the given mode, else HYC_ENOTSUP / HYC_EINVAL.  Pure host code. */
int hyc_check_shape(int64_t H, int32_t bits, int32_t group, int32_t mode);
/* bytes of one stored row: H*bits/8 */
int64_t hyc_stored_row_bytes(int64_t H, int32_t bits);
/* number of fp32 [H] partial rows hyc_rmsnorm_bwd needs in dw_partials for M tokens (an upper bound over all
 * descriptors), and the number it actually writes, rows [0, n), for one descriptor */
int64_t hyc_rmsnorm_bwd_partials(int64_t M, int64_t H);
int64_t hyc_rmsnorm_bwd_partial_rows(int64_t M, int64_t H, const hyc_desc* d);

/* ---- calibration, channel mode --------------------------------------------------------------- */
/* amax[c] = max(amax[c], max_m |x[m, c]|); the caller zero-fills amax (fp32 [H]) before the first call. */
int hyc_channel_absmax(const void* x, int64_t M, int64_t H, float* amax, void* stream);
/* the k largest amax, ties to the lower channel, written ascending to idx [k]; plan [H/8] as described above. */
int hyc_select_channels(const float* amax, int64_t H, int32_t k, int32_t* idx, uint32_t* plan, void* stream);

/* ---- calibration quantile ---------------------------------------------------------------------- */
/* out[0] = the k-th smallest (k = 1..n) of the n values of x (bf16 or fp32, HYC_DTYPE_*), as fp32; NaN sorts last,
 * -0 before +0.  workspace: hyc_kth_value_workspace_bytes() bytes of device memory, 16-byte aligned, any contents.
 * n < 2^31. */
int64_t hyc_kth_value_workspace_bytes(void);
int hyc_kth_value(const void* x, int32_t x_dtype, int64_t n, int64_t k, float* out, void* workspace, void* stream);

/* ---- standalone compress / decompress -------------------------------------------------------- */
/* x bf16 [M,H] -> stored; channel mode also writes vals [M,k] and scales [M,H/group];
 * threshold mode writes per-row outlier counts to row_counts (int32 [M], may be NULL). */
int hyc_compress(const void* x, int64_t M, int64_t H, const hyc_desc* d, void* stored, void* vals, void* scales,
                 int32_t* row_counts, void* stream);
/* the same for x whose rows are ldx >= H elements apart (a column slice of a wider matrix, e.g. one projection out
 * of a fused q/k/v GEMM); ldx a multiple of 8; channel scheme only (otherwise ldx must equal H) */
int hyc_compress_rows(const void* x, int64_t ldx, int64_t M, int64_t H, const hyc_desc* d, void* stored, void* vals,
                      void* scales, int32_t* row_counts, void* stream);
/* -> xhat bf16 [M,H]; channel mode reads vals/scales, threshold mode reads the CSR in the descriptor. */
int hyc_decompress(const void* stored, const void* vals, const void* scales, int64_t M, int64_t H, const hyc_desc* d,
                   void* xhat, void* stream);

/* ---- threshold-mode outliers as CSR ---------------------------------------------------------- */
/* counts[m] = #{c : |x[m,c] - base[m,c]| > threshold} */
int hyc_ref_outlier_count(const void* x, int64_t M, int64_t H, const hyc_desc* d, int32_t* counts, void* stream);
/* row_ptr int32 [M+1] = exclusive prefix sums of the counts (or hyc_csr_offsets with a capacity: row m then keeps its
 * first row_ptr[m+1] - row_ptr[m] outliers); fills cols / vals in ascending column order */
int hyc_ref_outlier_fill(const void* x, int64_t M, int64_t H, const hyc_desc* d, const int32_t* row_ptr,
                         int32_t* cols, void* vals, void* stream);

/* ---- RMSNorm ----------------------------------------------------------------------------------- */
/* y = bf16((x*rstd)*w), rstd = 1/sqrt(mean(x^2)+eps) [M] fp32, and x compressed as hyc_compress does. */
int hyc_rmsnorm_fwd_compress(const void* x, const void* w, int32_t w_dtype, float eps, int64_t M, int64_t H,
                             const hyc_desc* d, void* y, float* rstd, void* stored, void* vals, void* scales,
                             int32_t* row_counts, void* stream);
/* dx = (w*dy - (xn*c1 + c2))*rstd with xn = xhat*rstd, c1 = mean(xn*w*dy), c2 = c2_quirk ? mean(w*dy) : 0;
 * dw = sum_m dy*xn (fp32 accumulation, fixed order) written in w's dtype.  With dw == NULL the last step, the
 * column sum of the partial rows, is left to the caller (e.g. to accumulate over micro-batches first):
 * dw = sum of rows [0, hyc_rmsnorm_bwd_partial_rows(M, H, d)) of dw_partials. */
int hyc_rmsnorm_bwd(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                    int32_t w_dtype, const float* rstd, int64_t M, int64_t H, const hyc_desc* d, int32_t c2_quirk,
                    void* dx, float* dw_partials, void* dw, void* stream);

/* hyc_rmsnorm_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid allocation): the same kernels and results, but the fp32 partial rows of dw live in a device
 * array inside the library, so there is no dw_partials argument and the call allocates nothing.  It has no counterpart
 * in the reference.  Limits: hyc_rmsnorm_bwd_partial_rows(M, H, d) * H <= HYC_RMSNORM_BWD_STATIC_MAX_FLOATS (16 MiB of
 * fp32; with 2- or 4-bit codes every width up to 16384 channels fits at any M: at most 256 rows), HYC_EINVAL beyond; dw must not be
 * NULL.  Each GPU the library runs on holds its own 16 MiB array until the process ends; every call on a GPU uses that
 * GPU's array, so two calls that overlap on one GPU (different streams) race: serialise them or use hyc_rmsnorm_bwd.
 * The array used is the CURRENT device's: the current device must be the one that owns `stream` and the buffers.  The
 * first call on a device asks the runtime for the array's address (no allocation); that call must come outside a stream
 * capture (HYC_EINVAL under one) - a call with M = 0 does it and launches nothing. */
#define HYC_RMSNORM_BWD_STATIC_MAX_FLOATS (4 * 1024 * 1024)
int hyc_rmsnorm_bwd_static(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                           int32_t w_dtype, const float* rstd, int64_t M, int64_t H, const hyc_desc* d, int32_t c2_quirk,
                           void* dx, void* dw, void* stream);

/* LayerNorm forward with the compression of x fused in (efficient_layernorm.py:15-61 kernel, :203-260 Function):
 * mean = sum(x)/H, rstd = 1/sqrt(sum((x-mean)^2)/H + eps) (both fp32 [M]), y = bf16(((x-mean)*rstd)*w + b); bias may be
 * NULL, else it has w's dtype.  Other arguments as hyc_rmsnorm_fwd_compress.  Rows of at most 1024 chunks per segment
 * (H*bits/64 <= 1024), HYC_ENOTSUP beyond. */
int hyc_layernorm_fwd_compress(const void* x, const void* w, const void* bias, int32_t w_dtype, float eps, int64_t M,
                               int64_t H, const hyc_desc* d, void* y, float* mean, float* rstd, void* stored, void* vals,
                               void* scales, int32_t* row_counts, void* stream);

/* LayerNorm backward (efficient_layernorm.py:66-148, 262-330): xn = (xhat - mean)*rstd, dx as above with both
 * means (c1, c2), dw = sum_m dy*xn.  db = sum_m dy is a plain reduction left to the caller.  Buffers as for
 * hyc_rmsnorm_bwd. */
int hyc_layernorm_bwd(const void* dy, const void* stored, const void* vals, const void* scales, const void* w,
                      int32_t w_dtype, const float* mean, const float* rstd, int64_t M, int64_t H, const hyc_desc* d,
                      void* dx, float* dw_partials, void* dw, void* stream);

/* ---- activation backward ------------------------------------------------------------------- */
/* dx = act'(xhat) * g evaluated op by op in bf16 as the reference expressions are. */
int hyc_act_bwd(int32_t act, const void* g, const void* stored, const void* vals, const void* scales, int64_t M,
                int64_t H, const hyc_desc* d, void* dx, void* stream);
/* dx1 = g * x2hat, dx2 = x1hat * g */
int hyc_hadamard_bwd(const void* g, const void* stored1, const void* vals1, const void* scales1, const hyc_desc* d1,
                     const void* stored2, const void* vals2, const void* scales2, const hyc_desc* d2, int64_t M,
                     int64_t H, void* dx1, void* dx2, void* stream);

/* Backward of h = act(gate) * up (SwiGLU / GeGLU) in one pass over the three activations that
 * EfficientMemorySiLU/GELU (efficient_silu.py:11-53, efficient_gelu.py:11-64: saves gate) and EfficientMemoryHadamard
 * (efficient_hadamard.py:9-83: saves act(gate) and up) keep: d_up = a_hat * g, d_gate = act'(gate_hat) * bf16(g * up_hat).
 * Same results as hyc_hadamard_bwd followed by hyc_act_bwd; channel scheme, one code width for the three. */
int hyc_gated_act_bwd(int32_t act, const void* g, const void* stored_a, const void* vals_a, const void* scales_a,
                      const hyc_desc* d_a, const void* stored_u, const void* vals_u, const void* scales_u,
                      const hyc_desc* d_u, const void* stored_g, const void* vals_g, const void* scales_g,
                      const hyc_desc* d_g, int64_t M, int64_t H, void* d_gate, void* d_up, void* stream);

/* Forward of the same product with its three saves fused in: h = bf16(bf16(act(gate)) * up), plus the channel-compressed
 * forms of act(gate), up and gate (what EfficientMemorySiLU/GELU.forward, efficient_silu.py:13-40 / efficient_gelu.py:13-40,
 * and EfficientMemoryHadamard.forward, efficient_hadamard.py:11-53, compute and save), in one pass over gate and up;
 * act(gate) is never written to memory.  gate and up are bf16 [M, H] with row pitches ld_gate, ld_up (elements).  act:
 * HYC_ACT_SILU = F.silu; HYC_ACT_GELU_TANH = the GELU module, whose forward is the erf form (F.gelu) and whose backward
 * is the tanh form.  Same bytes as the separate calls; channel scheme, one code width (2, 4 or 8 bits) and group size (64
 * or 128) for the three, H * bits / 64 <= 768 (<= 512 with 2-bit codes), or up to 1024 when it divides by 2, 3 or 4 into
 * such parts of whole scale groups (H = 13824, 14336 and 16384 with 4-bit codes do); HYC_ENOTSUP otherwise (the separate
 * calls cover every shape). */
int hyc_gated_act_fwd(int32_t act, const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, int64_t M, int64_t H,
                      const hyc_desc* d_a, const hyc_desc* d_u, const hyc_desc* d_g, void* h, void* stored_a, void* vals_a,
                      void* scales_a, void* stored_u, void* vals_u, void* scales_u, void* stored_g, void* vals_g,
                      void* scales_g, void* stream);

/* The operators taken one at a time, forward with the save fused in (every operand read once; channel scheme; the same
 * bytes as the elementwise op followed by hyc_compress_rows):
 *   hyc_act_fwd_compress       y = act(x) and x compressed (EfficientMemorySiLU / GELU forward, efficient_silu.py:13-40,
 *                              efficient_gelu.py:13-40; act codes as for hyc_gated_act_fwd); 2-, 4- or 8-bit codes
 *   hyc_hadamard_fwd_compress  y = x1 * x2 and both operands compressed (EfficientMemoryHadamard forward,
 *                              efficient_hadamard.py:11-53); one code width (2, 4 or 8 bits) and group size for both
 * Inputs are bf16 [M, H] with row pitches in elements; groups of 64 or 128 channels, H * bits / 64 <= 1024 (<= 512 for
 * two operands of 2-bit codes); HYC_ENOTSUP otherwise. */
int hyc_act_fwd_compress(int32_t act, const void* x, int64_t ldx, int64_t M, int64_t H, const hyc_desc* d, void* y,
                         void* stored, void* vals, void* scales, void* stream);
int hyc_hadamard_fwd_compress(const void* x1, int64_t ld1, const void* x2, int64_t ld2, int64_t M, int64_t H,
                              const hyc_desc* d1, const hyc_desc* d2, void* y, void* stored1, void* vals1, void* scales1,
                              void* stored2, void* vals2, void* scales2, void* stream);

/* ---- softmax -------------------------------------------------------------------------------- */
/* x bf16 [rows, N] -> y = softmax(x, -1) bf16 and counts[r] = #{j : y[r,j] > bf16(threshold)} (counts may be
 * NULL).  With x == NULL, y is taken as given and only the counts are produced.  For N <= 4096 y may be x itself
 * (in place: a row is held in registers before any of it is written); the same holds for the causal form. */
int hyc_softmax_fwd(const void* x, int64_t rows, int64_t N, float threshold, void* y, int32_t* counts, void* stream);
/* the same with the causal attention mask built in (models/modeling_llama.py:452-459 adds it to the scores before the
 * softmax): row r is query position r % period and sees columns 0..position; columns beyond are not read and come
 * out as exact zeros.  1 <= period <= N <= 4096. */
int hyc_softmax_causal_fwd(const void* x, int64_t rows, int64_t N, int64_t period, float threshold, void* y,
                           int32_t* counts, void* stream);
/* Row offsets from per-row counts (of hyc_softmax_fwd, hyc_ref_outlier_count or the fused forwards), without the host:
 * row_ptr int32 [rows+1], row_ptr[r] = min(capacity, counts[0] + ... + counts[r-1]); *total (int64, may be NULL) = the
 * uncut sum.  capacity = the entries the caller's cols / vals buffers hold (negative: no limit).  With the offsets cut
 * off at a capacity, the fill entry points keep the first row_ptr[r+1] - row_ptr[r] entries of row r and drop the rest,
 * and every consumer reads exactly what was kept; total > capacity tells the caller that entries were dropped.  This is
 * what lets a calibrated caller size cols / vals ahead of time (e.g. 1.25 x the kept fraction it measured) instead of
 * reading the total back before it allocates, as the reference's to_sparse() does (compress_function.py:153, :269). */
int hyc_csr_offsets(const int32_t* counts, int64_t rows, int64_t capacity, int32_t* row_ptr, int64_t* total, void* stream);
/* the kept probabilities as CSR: row_ptr int32 [rows+1] (exclusive prefix sums of counts, or hyc_csr_offsets), cols
 * ascending per row; row r receives its first row_ptr[r+1] - row_ptr[r] kept entries */
int hyc_softmax_fill(const void* y, int64_t rows, int64_t N, float threshold, const int32_t* row_ptr, int32_t* cols,
                     void* vals, void* stream);
/* dx = (g - sum_j g_j*yh_j) * yh, yh = the CSR probabilities (zero elsewhere); dx may be g itself (in place) */
int hyc_softmax_bwd(const void* g, int64_t rows, int64_t N, const int32_t* row_ptr, const int32_t* cols,
                    const void* vals, void* dx, void* stream);
/* yh as a dense bf16 [rows, N] matrix */
int hyc_softmax_dense(int64_t rows, int64_t N, const int32_t* row_ptr, const int32_t* cols, const void* vals,
                      void* y_hat, void* stream);

/* ---- weight gradient ------------------------------------------------------------------------- */
/* out[n, h] = alpha * sum_m dy[m, n] * x_hat[m, h] + beta * out[n, h]; dy bf16 [M, N_out] with row stride ldy,
 * x_hat dequantised on the fly (channel mode) or read as bf16 (HYC_MODE_DENSE); out [N_out, H] bf16 or fp32.
 * workspace: hyc_gradw_workspace_bytes() bytes of device memory, 16-byte aligned (may be 0 -> NULL). */
int64_t hyc_gradw_workspace_bytes(int64_t M, int64_t N_out, int64_t H);
int hyc_gradw_gemm(const void* dy, int64_t ldy, const void* stored, const void* vals, const void* scales, int64_t M,
                   int64_t N_out, int64_t H, const hyc_desc* d, float alpha, float beta, void* out, int32_t out_dtype,
                   void* workspace, void* stream);

/* ---- low-rank base ----------------------------------------------------------------------------- */
/* out[m, :] = bf16(x[m, :] -/+ L[m mod S, :] @ R); L bf16 [S, rank], R bf16 [rank, H]; out may alias x */
int hyc_low_rank_update(const void* L, const void* R, const void* x, void* out, int64_t M, int64_t S, int64_t H,
                        int32_t rank, int32_t subtract, void* stream);

/* ---- rotary embedding + attention layout ----------------------------------------------------- */
/* x bf16 [B, S, heads, head_dim] (what the projections produce) -> the rotated tensor as [B, heads, S, head_dim] in
 * out_heads (what the batched attention GEMMs consume) and, when out_rows is not NULL, also in the input's layout
 * (apply_rotary_pos_emb, models/modeling_llama.py:236-260, with the .view().transpose(1, 2) of :423-425).
 *   y[i] = x[i] cos[i] - x[i+h] sin[i],  y[i+h] = x[i+h] cos[i+h] + x[i] sin[i+h],  h = head_dim / 2
 * cos / sin bf16 [S, head_dim]; both NULL = layout change only (the value tensor).  fp32 arithmetic, one rounding.
 * x_pitch = elements between consecutive tokens of x (heads*head_dim when x is contiguous; larger when x is a column
 * slice of a fused q/k/v projection).
 * hyc_rope_from_heads is the transpose: gradients [B, heads, S, head_dim] -> [B, S, heads, head_dim],
 *   dx[i] = g[i] cos[i] + g[i+h] sin[i+h],  dx[i+h] = g[i+h] cos[i+h] - g[i] sin[i].
 * head_dim a multiple of 16. */
int hyc_rope_to_heads(const void* x, int64_t x_pitch, const void* cosv, const void* sinv, int64_t B, int64_t S,
                      int64_t heads, int64_t head_dim, void* out_heads, void* out_rows, void* stream);
int hyc_rope_from_heads(const void* g, const void* cosv, const void* sinv, int64_t B, int64_t S, int64_t heads,
                        int64_t head_dim, void* out_rows, void* stream);

/* ---- seeded dropout ----------------------------------------------------------------------------- */
/* EfficientMemoryDropoutFunc, operators/efficient_dropout.py:56-79: the keep mask of element i is
 * tl.rand(seed, i) > p (Philox4x32-10, counter (i,0,0,0), key = the two words of seed), so nothing is saved.
 * backward == 0: out = keep ? bf16(x / (1-p)) : 0;  backward != 0: out = keep ? x : 0 (the reference's backward does
 * not rescale).  x, out bf16 [n], n < 2^31, 0 <= p < 1. */
int hyc_dropout(const void* x, void* out, int64_t n, float p, uint64_t seed, int32_t backward, void* stream);

/* ---- NF4 frozen base weights ------------------------------------------------------------------- */
/* Blocks of 64 consecutive weights: absmax[i] = max |w| of block i (fp32), packed byte j holds the level indices of
 * weights 2j (high nibble) and 2j+1 (low nibble); level index = nearest of the 16 NormalFloat4 levels to w / absmax.
 * n = number of weights, a multiple of 64.  w / out bf16 [n], packed uint8 [n/2], absmax fp32 [n/64].
 * out = bf16(level * absmax). */
int hyc_nf4_quantize(const void* w, int64_t n, void* packed, float* absmax, void* stream);
int hyc_nf4_dequantize(const void* packed, const float* absmax, int64_t n, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HYC_ABI_H */
