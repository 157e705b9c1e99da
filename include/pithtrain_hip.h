/*
 * C-ABI of libpithtrain_hip.so: hand-written gfx950 kernels for PithTrain's FP8
 * grouped-expert path.  Plain pointers and sizes only; every pointer is a device
 * pointer unless it says "host".  All launches go to `stream` (a hipStream_t passed
 * as void*); nothing here synchronises, allocates or frees device memory.
 *
 * Return value: 0 on success, negative PT_ERR_* otherwise; pt_last_error() gives a
 * thread-local message for the last failure.
 *
 * Each entry point names the reference interface it replaces
 * (paths relative to the PithTrain source tree).
 */
#ifndef PITHTRAIN_HIP_H
#define PITHTRAIN_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pt_stream_t;

enum { PT_OK = 0, PT_ERR_INVALID = -1, PT_ERR_LAUNCH = -2, PT_ERR_UNSUPPORTED = -3 };
/* element types of bf16/fp32/fp16 tensors */
enum { PT_BF16 = 0, PT_F32 = 1, PT_F16 = 2 };

const char* pt_last_error(void);
int pt_abi_version(void);

/* ------------------------------------------------------------------------------------------
 * Blockwise FP8 (e4m3fn) quantisation, power-of-two fp32 scales.
 * Replaces pithtrain/operators/deepgemm_quantize.py (six Triton kernels).
 * x is [M,N] with row stride ldx (elements) and unit column stride; dtype PT_BF16, PT_F16 or
 * PT_F32 (the reference's kernels load any float type and convert to fp32,
 * deepgemm_quantize.py:141-152).
 * ------------------------------------------------------------------------------------------ */

/* layout of the colwise twin written by pt_quant_rowwise_colwise */
enum {
  PT_CH_ROWMAJOR = 0,  /* ch_fp8[M,N],  ch_scale[M/128,N]   fp8cast_rowwise_colwise :204-259 */
  PT_CH_TRANSPOSED = 1,/* ch_fp8[N,M],  ch_scale[M/128,N]   (layout of this library's wgrad GEMM) */
  PT_CH_KMAJOR = 2     /* flat per-group (N,K_g) blocks, ch_scale[N,M/128]  fp8cast_rowwise_kmajor :262-333 */
};

/* 1x128 rowwise + 128-row colwise from one read.  M % 128 == 0 (deepgemm_quantize.py:219).
 * offs/num_groups (int32 inclusive row offsets, multiples of 128) give the PT_CH_KMAJOR layout its
 * groups.  For every layout, when offs is given, offs[num_groups-1] is the number of rows that
 * are quantised: M may then be an upper bound known on the host (buffers sized for the largest
 * row count a routing can produce) while the real count stays in device memory, and row tiles at
 * or past it are left untouched.  Without offs all M rows are quantised. */
int pt_quant_rowwise_colwise(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                             void* tok_fp8, float* tok_scale, void* ch_fp8, float* ch_scale,
                             int ch_layout, const int32_t* offs, int32_t num_groups,
                             pt_stream_t stream);

/* pt_quant_rowwise_colwise on gathered rows: output row r is quantised from source row
 * row_index[r] of x (a negative index gives an all-zero row: zero bytes, the scale of amax 0).
 * M counts output rows.  With row_index = the scatter's source map this is
 * fp8cast_rowwise_colwise(scatter_for_grouped_gemm(x)) without materialising the permuted bf16
 * copy (token_scatter.py:103-153 followed by deepgemm_quantize.py:204-259). */
int pt_quant_rowwise_colwise_rows(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                  const int32_t* row_index, void* tok_fp8, float* tok_scale,
                                  void* ch_fp8, float* ch_scale, int ch_layout,
                                  const int32_t* offs, int32_t num_groups, pt_stream_t stream);

/* SwiGLU fused into the activation quantisation (bf16 only).  Forward: h = bf16(silu(gate) * up)
 * with gate = gate_up[:, :half], up = gate_up[:, half:], quantised as pt_quant_rowwise_colwise
 * with the PT_CH_TRANSPOSED twin: tok_fp8[M,half], tok_scale[M,ceil(half/128)], ch_t_fp8[half,M],
 * ch_scale[M/128,half].  Same bits as silu_mul (silu_mul.py:28-49) followed by
 * fp8cast_rowwise_colwise (deepgemm_quantize.py:204-259); h itself is never written.
 * valid_rows (optional, device): *valid_rows rows are processed, the row tiles past them are left
 * untouched (M is then the host-side upper bound the buffers are sized for). */
int pt_silu_mul_quant_rowwise_colwise(const void* gate_up, int64_t M, int64_t half,
                                      int64_t ld_gate_up, void* tok_fp8, float* tok_scale,
                                      void* ch_t_fp8, float* ch_scale, const int32_t* valid_rows,
                                      pt_stream_t stream);
/* Backward twin: [dgate | dup] = silu_mul backward (silu_mul.py:52-87) of grad_h[M,half] at the
 * saved gate_up[M,2*half], rounded to bf16 and quantised to tok_fp8[M,2*half],
 * tok_scale[M,ceil(2*half/128)], ch_t_fp8[2*half,M], ch_scale[M/128,2*half]. */
int pt_silu_mul_bwd_quant_rowwise_colwise(const void* grad_h, int64_t ld_grad_h,
                                          const void* gate_up, int64_t ld_gate_up, int64_t M,
                                          int64_t half, void* tok_fp8, float* tok_scale,
                                          void* ch_t_fp8, float* ch_scale, const int32_t* valid_rows,
                                          pt_stream_t stream);
/* The same pair for the clamped SwiGLU of GPT-OSS (interleaved (gate, up) pairs, alpha, limit):
 * quantises h = clamped_swiglu(gate_up[M,2*half]) (clamped_swiglu.py:18-46) as
 * fp8cast_rowwise_colwise (deepgemm_quantize.py:204-259) would, without writing h:
 * tok_fp8[M,half], tok_scale[M,ceil(half/128)], ch_t_fp8[half,M], ch_scale[M/128,half]. */
int pt_clamped_swiglu_quant_rowwise_colwise(const void* gate_up, int64_t M, int64_t half,
                                            int64_t ld_gate_up, float alpha, float limit,
                                            void* tok_fp8, float* tok_scale, void* ch_t_fp8,
                                            float* ch_scale, const int32_t* valid_rows,
                                            pt_stream_t stream);
/* Backward twin: the gradient of gate_up in its interleaved layout (clamped_swiglu.py:49-89) from
 * grad_h[M,half], rounded to bf16 and quantised to tok_fp8[M,2*half], tok_scale[M,ceil(2*half/128)],
 * ch_t_fp8[2*half,M], ch_scale[M/128,2*half].  col_sum[M/128, 2*half] (fp32) receives the column
 * sums of every 128-row tile of the bf16 gradient: summed over a group's tiles (pt_segment_sum
 * with the group ends divided by 128) they are the bias gradient that _segment_sum_kernel
 * (indexed_bias_add.py:20-51) computes from the materialised gradient. */
int pt_clamped_swiglu_bwd_quant_rowwise_colwise(const void* grad_h, int64_t ld_grad_h,
                                                const void* gate_up, int64_t ld_gate_up, int64_t M,
                                                int64_t half, float alpha, float limit,
                                                void* tok_fp8, float* tok_scale, void* ch_t_fp8,
                                                float* ch_scale, float* col_sum,
                                                const int32_t* valid_rows, pt_stream_t stream);

/* rowwise(x) + rowwise(x^T): t_fp8[N,M], t_scale[N,ceil(M/128)].
 * fp8cast_rowwise_transpose, deepgemm_quantize.py:429-482 */
int pt_quant_rowwise_transpose(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                               void* tok_fp8, float* tok_scale, void* t_fp8, float* t_scale,
                               pt_stream_t stream);
/* The same with a row pitch ld_t >= M (bytes) for t_fp8: a reduction over all tokens reads the
 * transposed operand along rows, and a power-of-two pitch (M = 8192, 32768 tokens) puts those rows
 * on few memory channels.  No counterpart in the reference (its transposed outputs are packed). */
int pt_quant_rowwise_transpose_ld(const void* x, int dtype, int64_t M, int64_t N, int64_t ldx,
                                  void* tok_fp8, float* tok_scale, void* t_fp8, int64_t ld_t,
                                  float* t_scale, pt_stream_t stream);

/* rowwise(x) + 128x128 blockwise(x^T): blk_t_fp8[K,M], blk_t_scale[ceil(K/128),ceil(M/128)].
 * fp8cast_rowwise_blockwise_transpose, deepgemm_quantize.py:575-629 */
int pt_quant_rowwise_blockwise_transpose(const void* x, int dtype, int64_t M, int64_t K,
                                         int64_t ldx, void* tok_fp8, float* tok_scale,
                                         void* blk_t_fp8, float* blk_t_scale, pt_stream_t stream);
/* The same with a row pitch ld_t >= M (bytes) for blk_t_fp8 (see pt_quant_rowwise_transpose_ld). */
int pt_quant_rowwise_blockwise_transpose_ld(const void* x, int dtype, int64_t M, int64_t K,
                                            int64_t ldx, void* tok_fp8, float* tok_scale,
                                            void* blk_t_fp8, int64_t ld_t, float* blk_t_scale,
                                            pt_stream_t stream);

/* 128x128 blockwise(x) + blockwise(x^T) for x[G,N,K] (element strides stride_g, stride_row):
 * fp8[G,N,K], scale[G,ceil(N/128),ceil(K/128)], fp8_t[G,K,N], scale_t[G,ceil(K/128),ceil(N/128)].
 * fp8cast_blockwise_transpose (:709-756, G == 1) and fp8cast_blockwise_transpose_batched
 * (:846-899).  fp8_t and scale_t may both be NULL: then only fp8 and scale are written (the
 * transposed twin holds the same bytes and the transposed scale grid, and pt_gemm_m_grouped_nn
 * reads the forward layout directly). */
int pt_quant_blockwise_transpose_batched(const void* x, int dtype, int64_t G, int64_t N, int64_t K,
                                         int64_t stride_g, int64_t stride_row, void* fp8,
                                         float* scale, void* fp8_t, float* scale_t,
                                         pt_stream_t stream);
/* The same into slices of larger outputs: group strides for fp8 / scale, and for the transposed
 * twin its row pitch t_ld (>= N), group stride, and the row length scale_t_ld of its scale grid.
 * Separate gate and up weights are quantised into one fused [G, 2I, K] operand this way (the up
 * half starts I rows, i.e. I*K bytes / I columns of the twin, further in). */
int pt_quant_blockwise_transpose_batched_into(const void* x, int dtype, int64_t G, int64_t N,
                                              int64_t K, int64_t stride_g, int64_t stride_row,
                                              void* fp8, int64_t fp8_stride_g, float* scale,
                                              int64_t scale_stride_g, void* fp8_t, int64_t t_ld,
                                              int64_t t_stride_g, float* scale_t,
                                              int64_t scale_t_ld, int64_t scale_t_stride_g,
                                              pt_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * FP8 GEMMs (fp32 accumulate on the MFMA units, scales applied in hardware as E8M0).
 * Replace the DeepGEMM call sites of pithtrain/operators/linear.py and grouped_linear.py.
 * ------------------------------------------------------------------------------------------ */

/* out[m,n] = sum_k a[m,k] b[n,k];  a_scale[M,ceil(K/128)] (1x128), b_scale[ceil(N/128),ceil(K/128)]
 * (128x128).  out is bf16 [M,N] (out_dtype PT_BF16) or fp32 (PT_F32).
 * deep_gemm.fp8_fp4_gemm_nt at linear.py:40 (forward :57, dgrad :77, wgrad :80). */
int pt_gemm_nt_dense(const void* a_fp8, const float* a_scale, const void* b_fp8,
                     const float* b_scale, void* out, int out_dtype, int64_t M, int64_t N,
                     int64_t K, pt_stream_t stream);
/* The same for operands with row pitches lda, ldb >= K (bytes, multiples of 16): the padded
 * transposed operands of pt_quant_rowwise_transpose_ld / pt_quant_rowwise_blockwise_transpose_ld. */
int pt_gemm_nt_dense_ld(const void* a_fp8, int64_t lda, const float* a_scale, const void* b_fp8,
                        int64_t ldb, const float* b_scale, void* out, int out_dtype, int64_t M,
                        int64_t N, int64_t K, pt_stream_t stream);
/* Split-K form of pt_gemm_nt_dense for outputs with too few 256 x 256 tiles to fill the GPU (the
 * weight gradient of a dense linear, linear.py:61-83: M, N = weight dims, K = tokens): the
 * reduction is cut into `splits` ranges of split_len (a multiple of 128), range s is reduced into
 * the fp32 slab partial[s] ([splits, M, N], caller-provided), and pt_sum_partials adds the slabs
 * in the order of s and stores the sum as out_dtype (n = M * N, a multiple of 8). */
int pt_gemm_nt_dense_splitk(const void* a_fp8, const float* a_scale, const void* b_fp8,
                            const float* b_scale, float* partial, int32_t splits, int64_t split_len,
                            int64_t M, int64_t N, int64_t K, pt_stream_t stream);
int pt_gemm_nt_dense_splitk_ld(const void* a_fp8, int64_t lda, const float* a_scale,
                               const void* b_fp8, int64_t ldb, const float* b_scale, float* partial,
                               int32_t splits, int64_t split_len, int64_t M, int64_t N, int64_t K,
                               pt_stream_t stream);
int pt_sum_partials(const float* partial, int32_t splits, int64_t n, void* out, int out_dtype,
                    pt_stream_t stream);

/* Rows [offs[g-1], offs[g]) of a[M,K] use b[g] of b[G,N,K]; every offs[g] is a multiple of 128.
 * Rows at or past offs[G-1] are not written.  out bf16 [M,N].
 * deep_gemm.m_grouped_fp8(_fp4)_gemm_nt_contiguous at grouped_linear.py:88-101 (forward :146-154,
 * dgrad :192-200). */
int pt_gemm_m_grouped_nt(const void* a_fp8, const float* a_scale, const void* b_fp8,
                         const float* b_scale, void* out, int out_dtype, const int32_t* offs,
                         int32_t num_groups, int64_t M, int64_t N, int64_t K, pt_stream_t stream);

/* pt_gemm_m_grouped_nt whose result row r is written to out[out_row_index[r], :] (negative
 * index: the row is dropped); out is bf16 [out_rows, N], N % 8 == 0.  With out_row_index = the
 * scatter's source map this is padded_index_gather(gemm(...), reverse) - the un-permute of
 * token_scatter.py:297-309 (forward) or ScatterForGroupedGemm.backward (:271-284, dgrad) -
 * without the intermediate [M, N] tensor. */
int pt_gemm_m_grouped_nt_scatter(const void* a_fp8, const float* a_scale, const void* b_fp8,
                                 const float* b_scale, void* out, int out_dtype,
                                 const int32_t* offs, int32_t num_groups, int64_t M, int64_t N,
                                 int64_t K, const int32_t* out_row_index, int64_t out_rows,
                                 pt_stream_t stream);

/* pt_gemm_m_grouped_nt with the b operand given reduction-major: b[g] is [K, N] (K = the reduction,
 * row pitch N, N % 16 == 0) with scales [ceil(K/128), ceil(N/128)], i.e. a weight and its
 * 128 x 128 block scales as the forward pass stores them, read by the input-gradient GEMM
 * dX = dY W without the transposed FP8 copy of W that the call at grouped_linear.py:192-200 is given
 * (made by fp8cast_blockwise_transpose_batched, deepgemm_quantize.py:419-456).  Same products, same
 * order of accumulation, same bits as pt_gemm_m_grouped_nt on the transposed operand.  The _scatter
 * form stores result row r to out[out_row_index[r], :] like pt_gemm_m_grouped_nt_scatter. */
int pt_gemm_m_grouped_nn(const void* a_fp8, const float* a_scale, const void* b_fp8,
                         const float* b_scale, void* out, int out_dtype, const int32_t* offs,
                         int32_t num_groups, int64_t M, int64_t N, int64_t K, pt_stream_t stream);
int pt_gemm_m_grouped_nn_scatter(const void* a_fp8, const float* a_scale, const void* b_fp8,
                                 const float* b_scale, void* out, int out_dtype,
                                 const int32_t* offs, int32_t num_groups, int64_t M, int64_t N,
                                 int64_t K, const int32_t* out_row_index, int64_t out_rows,
                                 pt_stream_t stream);

/* pt_gemm_m_grouped_nt followed by `out + bias[group of the row]` in the output type (the result
 * is rounded to bf16, then the bias row of its group is added and the sum rounded again): the
 * grouped linear and the indexed_bias_add after it (models/gpt_oss.py:151-156,
 * indexed_bias_add.py:100-104) as one kernel.  bias is [G,N] bf16; N % 8 == 0. */
int pt_gemm_m_grouped_nt_bias(const void* a_fp8, const float* a_scale, const void* b_fp8,
                              const float* b_scale, void* out, int out_dtype, const int32_t* offs,
                              int32_t num_groups, int64_t M, int64_t N, int64_t K,
                              const void* bias, pt_stream_t stream);
/* Both of the above: the bias row of the group is added to the rounded result and the row is
 * stored at out[out_row_index[r]] (grouped linear + indexed_bias_add + the un-permuting
 * padded_index_gather of forward_stage3, models/gpt_oss.py:155-156,318-321, as one kernel). */
int pt_gemm_m_grouped_nt_scatter_bias(const void* a_fp8, const float* a_scale, const void* b_fp8,
                                      const float* b_scale, void* out, int out_dtype,
                                      const int32_t* offs, int32_t num_groups, int64_t M, int64_t N,
                                      int64_t K, const int32_t* out_row_index, int64_t out_rows,
                                      const void* bias, pt_stream_t stream);

/* dW[g][n,k] = sum_{m in group g} dY[m,n] X[m,k] with colwise-quantised operands stored
 * transposed: dy_t[N,M] and x_t[K,M] (PT_CH_TRANSPOSED) and their scales dy_scale[M/128,N],
 * x_scale[M/128,K].  out is [G,N,K]:
 *   out_dtype PT_F32 : fp32, accumulate==0 overwrites, !=0 adds (the `c=` operand)
 *   out_dtype PT_BF16: bf16(sum) rounded once; accumulate!=0 then adds the existing bf16 value
 *                      in fp32 and rounds again (weight.grad += wgrad.to(bf16)).
 * Groups with no rows get zeros (or are left unchanged when accumulating).
 * deep_gemm.k_grouped_fp8_gemm_{tn,nt}_contiguous + grad_weight_fn, grouped_linear.py:202-221. */
int pt_gemm_k_grouped_wgrad(const void* dy_t_fp8, const float* dy_scale, const void* x_t_fp8,
                            const float* x_scale, void* out, int out_dtype, int accumulate,
                            const int32_t* offs, int32_t num_groups, int64_t M, int64_t N,
                            int64_t K, pt_stream_t stream);
/* The same with the row length of the two scale arrays given: dy_scale[M/128, ld_dy_scale] and
 * x_scale[M/128, ld_x_scale] may be column slices of wider arrays (the gate and up halves of a
 * fused projection's colwise twin get their own weight-gradient tensors this way). */
int pt_gemm_k_grouped_wgrad_ld(const void* dy_t_fp8, const float* dy_scale, int64_t ld_dy_scale,
                               const void* x_t_fp8, const float* x_scale, int64_t ld_x_scale,
                               void* out, int out_dtype, int accumulate, const int32_t* offs,
                               int32_t num_groups, int64_t M, int64_t N, int64_t K,
                               pt_stream_t stream);

/* Which GEMM kernel the three entry points above launch: "auto" (or NULL: per call from the
 * shape; the default unless the environment variable PT_GEMM_IMPL names one of the others),
 * "p0" persistent kernel with the two-phase main loop, "q0" / "q1" persistent kernel with the
 * software-pipelined main loop (8 / 4 waves per workgroup), "t" one 128x128 tile per workgroup.
 * Every choice computes the same function; this exists for measurements and for tests that
 * cover each kernel.  Process-wide, not synchronised with concurrent GEMM calls.
 * No counterpart in the reference (DeepGEMM selects its kernels internally). */
int pt_gemm_select_kernel(const char* name);

/* ------------------------------------------------------------------------------------------
 * Routing-driven permute / unpermute.  Replace pithtrain/operators/token_scatter.py.
 * ------------------------------------------------------------------------------------------ */

/* Bytes of workspace pt_group_rows needs for m keys and num_groups groups. */
int64_t pt_group_rows_workspace_bytes(int64_t m, int32_t num_groups);

/* Stable counting sort of rows by group with every group padded to `alignment` rows.
 *   keys[m] int64 in [0,num_groups)            (expert_idxs)
 *   offs[G] int32 inclusive cumsum of padded sizes, ks[G] int32 padded sizes
 *   reverse[m] int64: destination row of source row i  (reverse_shuffle_idxs)
 *   src_of[cap] int32: source row of destination row r, -1 for pad rows (r < cap)
 * Canonical order: ascending source row inside a group.  Keys are expected in [0,num_groups); a row
 * whose key is outside belongs to no group: no src_of entry names it and its reverse entry is 0.
 * _compute_group_offsets_kernel + slot assignment of _scatter_for_grouped_gemm_kernel,
 * token_scatter.py:38-101. */
int pt_group_rows(const int64_t* keys, int64_t m, int32_t num_groups, int32_t alignment,
                  int32_t* offs, int32_t* ks, int64_t* reverse, int32_t* src_of, int64_t cap,
                  void* workspace, int64_t workspace_bytes, pt_stream_t stream);

/* pt_group_rows for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments, results and errors, but
 * the workspace is a device array built into the library (one copy per GPU, held until the
 * process ends) instead of an argument, and the call allocates and frees nothing.  It refuses
 * problems whose pt_group_rows_workspace_bytes(m, num_groups) exceeds
 * PT_GROUP_ROWS_STATIC_MAX_WORKSPACE (e.g. up to 262144 keys in 256 groups, or 524288 keys in 128).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and need nothing cleared in between.
 * The first call on a device looks the array's address up (hipGetSymbolAddress, which may load the
 * code object) and must be made outside a graph capture; a captured call records that one
 * address, so two graphs that contain it must not replay at the same time on one GPU either.
 * No counterpart in the reference, which allocates its counters with torch on every call
 * (token_scatter.py:205-207). */
#define PT_GROUP_ROWS_STATIC_MAX_WORKSPACE ((1 << 20) + 8192)
int pt_group_rows_static(const int64_t* keys, int64_t m, int32_t num_groups, int32_t alignment,
                         int32_t* offs, int32_t* ks, int64_t* reverse, int32_t* src_of, int64_t cap,
                         pt_stream_t stream);

/* out[r,:] = src_of[r] >= 0 ? in[pre ? pre[src_of[r]] : src_of[r], :] : 0   for r < rows_out,
 * where rows_out = min(cap, round_up(offs_last[0], tail_alignment)) read on the device when
 * offs_last != NULL, else cap.  Rows in [rows_out, cap) are not touched.  elem_bytes-wide
 * elements, H per row.  `pre` (int64, may be NULL) composes a first gather (the dedup expand)
 * into the same pass.
 * Row copy + pad/tail zeroing of _scatter_for_grouped_gemm_kernel, token_scatter.py:103-153. */
int pt_permute_rows(const void* in, int64_t ld_in, void* out, int64_t ld_out, const int32_t* src_of,
                    const int64_t* pre, const int32_t* offs_last, int32_t tail_alignment,
                    int64_t cap, int64_t H, int32_t elem_bytes, pt_stream_t stream);

/* out[i,:] = in[index[i],:], i < n.  index int64.
 * _PaddedIndexGather.forward (token_scatter.py:297-309), ScatterForGroupedGemm.backward
 * (:271-284). */
int pt_gather_rows(const void* in, int64_t ld_in, void* out, int64_t ld_out, const int64_t* index,
                   int64_t n, int64_t H, int32_t elem_bytes, pt_stream_t stream);

/* Bytes of workspace pt_gather_rows_backward needs. */
int64_t pt_gather_rows_backward_workspace_bytes(int64_t n, int64_t rows);

/* grad_in[r,:] = sum over {j : index[j] == r} of grad_out[j,:], r < rows; summed in fp32 in
 * ascending j, rounded once to the element type (dtype PT_BF16 / PT_F32 / PT_F16).
 * _PaddedIndexGather.backward (scatter_add_), token_scatter.py:311-325. */
int pt_gather_rows_backward(const void* grad_out, int64_t ld_go, void* grad_in, int64_t ld_gi,
                            const int64_t* index, int64_t n, int64_t rows, int64_t H, int dtype,
                            void* workspace, int64_t workspace_bytes, pt_stream_t stream);

/* group_ids[r] = min(#{g : offs[g] <= r}, G-1), r < M; out_dtype_bytes 4 (int32) or 8 (int64).
 * precompute_group_indices, token_scatter.py:370-384; GptOssExperts.forward,
 * models/gpt_oss.py:146-150. */
int pt_group_indices(const int32_t* offs, int32_t num_groups, int64_t M, void* group_ids,
                     int32_t out_dtype_bytes, pt_stream_t stream);
/* out[r] = expand_idx[row_map[r]] (int32) where row_map[r] is in [0, n_expand) and the result in
 * [0, n_src), -1 otherwise.  Composes the scatter's source map with the dedup expand index
 * (models/qwen3_moe.py:222-224 gathers through expand_idx, then scatters), so that the first
 * quantisation of the expert block reads the deduplicated rows directly. */
int pt_compose_row_map(const int32_t* row_map, int64_t n, const int64_t* expand_idx,
                       int64_t n_expand, int64_t n_src, int32_t* out, pt_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Expert-parallel dispatch index construction with token dedup.
 * Replace the Triton kernels of pithtrain/operators/ep_dispatch.py.
 * ------------------------------------------------------------------------------------------ */

int64_t pt_dedup_workspace_bytes(int64_t m, int32_t k, int32_t num_experts, int32_t ep_size);

/* topk_ids[m,k] int64 (row stride ld_ids) -> tokens_per_ep_rank[ep], dedup_tokens_per_gpu[ep],
 * dispatch_token_idxs[m*ep] (first sum(dedup) valid), idxs[m*k], expand_idx[m*k],
 * send_meta[ep*(epr+1)], all int64.  Canonical order: ascending flat index inside an expert
 * bucket, ascending token id inside an EP-rank chunk.
 * fused_dedup_prepare_dispatch, ep_dispatch.py:271-420. */
int pt_dedup_prepare_dispatch(const int64_t* topk_ids, int64_t ld_ids, int64_t m, int32_t k,
                              int32_t num_experts, int32_t ep_size, int32_t experts_per_rank,
                              int64_t* tokens_per_ep_rank, int64_t* dedup_tokens_per_gpu,
                              int64_t* dispatch_token_idxs, int64_t* idxs, int64_t* expand_idx,
                              int64_t* send_meta, void* workspace, int64_t workspace_bytes,
                              pt_stream_t stream);

/* expert_idxs[s] = e % experts_per_rank for slot s in bucket e (s < sum(counts), s < max_total);
 * output_splits[g] = sum of counts of rank g.   build_expert_idxs, ep_dispatch.py:426-508. */
int pt_build_expert_idxs(const int64_t* tokens_per_expert_group, int32_t num_experts,
                         int32_t ep_size, int32_t experts_per_rank, int64_t max_total,
                         int64_t* expert_idxs, int64_t* output_splits, pt_stream_t stream);

/* out[i] = received[i] + exclusive_cumsum(dedup_counts)[sender(i)], sender from output_splits.
 * dedup_counts has element stride dedup_stride.   adjust_expand_idx, ep_dispatch.py:511-576. */
int pt_adjust_expand_idx(const int64_t* received, int64_t* out, const int64_t* dedup_counts,
                         int64_t dedup_stride, const int64_t* output_splits, int32_t ep_size,
                         int64_t n, pt_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Fused epilogues.  dtype is the storage type (PT_BF16 / PT_F16 / PT_F32); math in fp32.
 * ------------------------------------------------------------------------------------------ */

/* out = silu(gate) * up over n elements.   _silu_mul_fwd_kernel, silu_mul.py:28-49 */
int pt_silu_mul_fwd(const void* gate, const void* up, void* out, int64_t n, int dtype,
                    pt_stream_t stream);
/* _silu_mul_bwd_kernel, silu_mul.py:52-87 */
int pt_silu_mul_bwd(const void* grad_out, const void* gate, const void* up, void* grad_gate,
                    void* grad_up, int64_t n, int dtype, pt_stream_t stream);
/* The same two kernels on [rows, cols] views with their own leading dimensions (in elements), so
 * that the halves of a fused gate_up buffer are read in place and both gradients land in one
 * [rows, 2*cols] buffer: replaces the .contiguous() copies around silu_mul in
 * Qwen35MoeExperts.forward (models/qwen35_moe.py:196-199) and their autograd backward. */
int pt_silu_mul_fwd_2d(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* out,
                       int64_t ld_out, int64_t rows, int64_t cols, int dtype, pt_stream_t stream);
int pt_silu_mul_bwd_2d(const void* grad_out, int64_t ld_grad_out, const void* gate, int64_t ld_gate,
                       const void* up, int64_t ld_up, void* grad_gate, int64_t ld_grad_gate,
                       void* grad_up, int64_t ld_grad_up, int64_t rows, int64_t cols, int dtype,
                       pt_stream_t stream);
/* gate_up[M,2N] interleaved -> out[M,N]; n = M*N.  _clamped_swiglu_fwd_kernel,
 * clamped_swiglu.py:18-46 */
int pt_clamped_swiglu_fwd(const void* gate_up, void* out, int64_t n, float alpha, float limit,
                          int dtype, pt_stream_t stream);
/* _clamped_swiglu_bwd_kernel, clamped_swiglu.py:49-89 */
int pt_clamped_swiglu_bwd(const void* grad_out, const void* gate_up, void* grad_gate_up, int64_t n,
                          float alpha, float limit, int dtype, pt_stream_t stream);
/* out[r,:] = x[r,:] + bias[group_ids[r],:]  (group_ids int64).  _IndexedBiasAdd.forward,
 * indexed_bias_add.py:100-104 */
int pt_indexed_bias_add_fwd(const void* x, const void* bias, const int64_t* group_ids, void* out,
                            int64_t M, int64_t H, int dtype, pt_stream_t stream);
/* out[g,:] = sum of rows [offs[g-1], min(offs[g],M)) of x, fp32 accumulate, stored as out_dtype.
 * _segment_sum_kernel, indexed_bias_add.py:20-96 */
int pt_segment_sum(const void* x, const int32_t* offs, int32_t num_groups, void* out, int64_t M,
                   int64_t H, int dtype, int out_dtype, pt_stream_t stream);
/* The same sums with grouped row r read from x[row_index[r]] (x [x_rows,H] un-permuted; a negative
 * index is a padding row): the bias gradient of a grouped linear whose output rows were stored
 * through row_index, in the grouped order of the rows (same bits as gathering first). */
int pt_segment_sum_rows(const void* x, int64_t x_rows, const int32_t* row_index, const int32_t* offs,
                        int32_t num_groups, void* out, int64_t M, int64_t H, int dtype,
                        int out_dtype, pt_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Top-k weighted combine with the residual: the memory-bound step that follows the expert path.
 * forward_stage5, single-rank branch (models/qwen3_moe.py:229-237; the same expression in
 * models/deepseek_v2.py, models/gpt_oss.py, models/qwen35_moe.py).
 * ------------------------------------------------------------------------------------------ */

/* out[t,:] = residual[t,:] + S(sum_j float(moe[t*k+j,:]) * topk_weight[t,j]): fp32 products added in
 * the order j = 0..k-1, the sum rounded to the storage type S (dtype), the addition rounded again.
 * moe is [T*k,H], residual and out [T,H] (leading dimensions in elements), topk_weight fp32 [T,k],
 * 1 <= k <= 16.  residual may be NULL: out is then the rounded sum itself, the weighted sum that
 * ends the single-device MoE forward (models/qwen3_moe.py:119). */
int pt_moe_combine_fwd(const void* moe, int64_t ld_moe, const float* topk_weight,
                       const void* residual, int64_t ld_res, void* out, int64_t ld_out, int64_t T,
                       int32_t k, int64_t H, int dtype, pt_stream_t stream);
/* d_moe[t*k+j,:] = S(float(grad_out[t,:]) * topk_weight[t,j]);
 * d_weight[t,j] = sum_h grad_out[t,h] * moe[t*k+j,h] in fp32 (fixed reduction order);
 * the gradient of the residual is grad_out itself. */
int pt_moe_combine_bwd(const void* grad_out, int64_t ld_go, const void* moe, int64_t ld_moe,
                       const float* topk_weight, void* d_moe, int64_t ld_dmoe, float* d_weight,
                       int64_t T, int32_t k, int64_t H, int dtype, pt_stream_t stream);

/* Expert-parallel branch of forward_stage5 (models/qwen3_moe.py:238-245, same lines in
 * deepseek_v2.py:351-357, qwen35_moe.py:334-340, gpt_oss.py:334-340): row r of moe [rows,H] belongs
 * to the flat top-k slot local_idxs[r] (token local_idxs[r] / k), every weighted row is rounded to
 * S and added to a zeroed S accumulator, the residual is added last.  The reference's scatter_add_
 * leaves the order of the adds to the device's atomics; here a token's rows are added in ascending
 * r, every partial sum rounded to S (the result of a sequential scatter_add_).
 *
 * pt_moe_combine_ep_index: slot_row[s] = r for s = local_idxs[r], -1 for slots without a row
 * (slot_row int32 [slots], slots = T*k; entries of local_idxs must be distinct, values outside
 * [0, slots) are ignored). */
int pt_moe_combine_ep_index(const int64_t* local_idxs, int64_t rows, int64_t slots,
                            int32_t* slot_row, pt_stream_t stream);
int pt_moe_combine_ep_fwd(const void* moe, int64_t ld_moe, int64_t rows, const int32_t* slot_row,
                          const float* topk_weight, const void* residual, int64_t ld_res, void* out,
                          int64_t ld_out, int64_t T, int32_t k, int64_t H, int dtype,
                          pt_stream_t stream);
/* d_moe[r,:] = S(float(grad_out[t,:]) * topk_weight[t,j]) for r = slot_row[t*k+j];
 * d_weight[t,j] = sum_h grad_out[t,h] * moe[r,h] in fp32, 0 for a slot without a row. */
int pt_moe_combine_ep_bwd(const void* grad_out, int64_t ld_go, const void* moe, int64_t ld_moe,
                          int64_t rows, const int32_t* slot_row, const float* topk_weight,
                          void* d_moe, int64_t ld_dmoe, float* d_weight, int64_t T, int32_t k,
                          int64_t H, int dtype, pt_stream_t stream);

/* Router gate after the logits GEMM: softmax + top-k + weights of the chosen experts, one launch.
 *   mode 0: Qwen3MoeGate.forward (models/qwen3_moe.py:81-88), Qwen35MoeTopKRouter.forward
 *           (models/qwen35_moe.py:216-222) and DeepSeekV2MoEGate.forward (models/deepseek_v2.py:
 *           149-164): scores = softmax(logits) in fp32; with num_group > 1 only the topk_group
 *           groups of E/num_group contiguous experts with the largest maximum keep their scores
 *           (group_limited_greedy), the rest become 0; top-k of the scores; w = scores[topk_idx];
 *           w /= sum(w) if norm_topk_prob; w *= scale (routed_scaling_factor).
 *   mode 1: GptOssTopKRouter.forward (models/gpt_oss.py:176-182): top-k of the logits, then
 *           w = softmax(logits[topk_idx]) in fp32.
 * logits [T,E] in dtype (leading dimension in elements), E <= 512, k <= min(32, E).  topk_idx int64
 * [T,k] comes out sorted by descending value, ties to the lower expert index (torch.topk leaves
 * both open for sorted=False).  forced_idx (router replay, the `router_replay` hook of the same
 * functions) replaces the selection when not null.  scores fp32 [T,E] (what the load-balance loss
 * reads: after the group limit in mode 0, the full softmax in mode 1) is written when not null. */
int pt_router_topk_fwd(const void* logits, int64_t ld_logits, int dtype, int64_t T, int32_t E,
                       int32_t k, int mode, int norm_topk_prob, float scale, int32_t num_group,
                       int32_t topk_group, const int64_t* forced_idx, int64_t* topk_idx,
                       float* topk_weight, float* scores, pt_stream_t stream);
/* Gradient of the logits from d_weight fp32 [T,k] (and d_scores fp32 [T,E] when not null), through
 * the scale, the normalisation, the gather at topk_idx, the group limit and the softmax; the
 * scores are recomputed from the logits.  d_logits [T,E] in dtype. */
int pt_router_topk_bwd(const void* logits, int64_t ld_logits, int dtype, int64_t T, int32_t E,
                       int32_t k, int mode, int norm_topk_prob, float scale, int32_t num_group,
                       int32_t topk_group, const int64_t* topk_idx, const float* d_weight,
                       const float* d_scores, void* d_logits, int64_t ld_dlogits,
                       pt_stream_t stream);

/* In-place fused cross-entropy with mean reduction (CrossEntropy.forward and its Triton kernel
 * cross_entropy_fwd, operators/cross_entropy.py:16-78,86-118): logits [N,V] in dtype are
 * overwritten with the gradient of the mean loss, S((exp(x - max) / sum) / n) and, at the target,
 * S(float(stored) - 1/n), with n = max(1, number of rows whose target is not ignore_index); rows
 * with the ignored target become zero.  loss_rows fp32 [N] receives -(x_y - max - log sum) (0 for
 * ignored rows, NaN for a target outside [0, V)), loss fp32 [1] their sum over n, n_non_ignore
 * int64 [1] n itself.  Three launches on the stream, no host synchronisation. */
int pt_cross_entropy_fwd(void* logits, int64_t ld, int dtype, const int64_t* target, int64_t N,
                         int64_t V, int64_t ignore_index, float* loss_rows, float* loss,
                         int64_t* n_non_ignore, pt_stream_t stream);
/* CrossEntropy.backward (operators/cross_entropy.py:120-124): the stored gradient times the
 * incoming scalar (fp32 on the device, rounded to dtype first), in place. */
int pt_cross_entropy_bwd(void* grad, int64_t ld, int dtype, int64_t N, int64_t V,
                         const float* grad_output, pt_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PITHTRAIN_HIP_H */
