/*
 * fluxmi.h — C-ABI of the MI355X (gfx950) kernels behind Flux's single-GPU MoE operators.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream (passed as `void*`, i.e. a
 * `hipStream_t`; NULL = the default stream).  Nothing here allocates device memory: scratch space is
 * caller-provided (`workspace`, sized by the matching `*_workspace_bytes` call).  All calls are
 * asynchronous with respect to the host and never synchronise the stream.  Return value: 0 on success,
 * a negative `fluxmi_status` otherwise; `fluxmi_last_error()` gives a thread-local message.
 *
 * Citations name the interface of the reference (bytedance/flux) that each entry point stands in for.
 */
#ifndef FLUXMI_H_
#define FLUXMI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum fluxmi_status {
  FLUXMI_OK = 0,
  FLUXMI_ERR_INVALID_ARG = -1, /* null pointer, negative size, misaligned pointer, bad enum */
  FLUXMI_ERR_UNSUPPORTED = -2, /* shape / dtype combination no kernel covers */
  FLUXMI_ERR_WORKSPACE = -3,   /* workspace missing or too small */
  FLUXMI_ERR_HIP = -4          /* a HIP runtime call or kernel launch failed */
} fluxmi_status;

typedef enum fluxmi_dtype {
  FLUXMI_BF16 = 0,     /* bfloat16 operands, fp32 accumulate, bf16 (or fp32) output */
  FLUXMI_FP8_E4M3 = 1, /* OCP e4m3 (torch.float8_e4m3fn) operands, fp32 accumulate, bf16 (or fp32) output */
  FLUXMI_FP16 = 2      /* IEEE half operands, fp32 accumulate, fp16 (or fp32) output: the reference's fp16 variants of
                          both MoE ops (src/generator/gen_moe_ag_scatter.cc:26-39, gen_moe_gather_rs.cc:25-45) */
} fluxmi_dtype;

/* Library version (major*10000 + minor*100 + patch) and the last error text of the calling thread. */
int fluxmi_version(void);
const char *fluxmi_last_error(void);

/* Number of compute units of the current device (persistent kernels launch one workgroup per CU). */
int fluxmi_device_cu_count(void);

/* ------------------------------------------------------------------------------------------------
 * Routing: stable counting sort of (token, k) pairs by expert id.
 *
 * Stands in for `torch.bincount` + `calc_scatter_index_stable` + `calc_gather_index`
 * (python/flux/testing/moe_utils.py:141-144, :96-138, :215-217) and for the device kernels
 * `calc_scatter_index` (src/cuda/moe_utils.cu:23-75) and `calc_gather_index_impl`
 * (src/moe_ag_scatter/sort_util.cu:39-92, :121-160), with the *stable* order as the contract:
 *   splits[e]          = #{i : choosed[i] == e}
 *   offsets            = exclusive prefix sum of splits, offsets[E] = number of routed pairs
 *   scatter_index[i]   = offsets[choosed[i]] + #{i' < i : choosed[i'] == choosed[i]}
 *   gather_index[scatter_index[i]] = i / topk,   topk_index[scatter_index[i]] = i % topk
 * `choosed` holds ntokens*topk int32 in [0, nexperts); ids outside that range are treated as dropped
 * pairs: they get scatter_index -1 and take no row.  Any of the output pointers except
 * `scatter_index` may be NULL.
 * ---------------------------------------------------------------------------------------------- */
size_t fluxmi_moe_route_sort_workspace_bytes(int32_t ntokens, int32_t topk, int32_t nexperts);
int fluxmi_moe_route_sort(const int32_t *choosed, int32_t ntokens, int32_t topk, int32_t nexperts,
                          int32_t *splits, int32_t *offsets, int32_t *scatter_index,
                          int32_t *gather_index, int32_t *topk_index, void *workspace,
                          size_t workspace_bytes, void *stream);

/* The same sort for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The scratch the sort needs lives
 * in a device array inside the library (fluxmi_moe_route_sort_static_max_bytes() = 4 MiB per GPU, held until
 * the process ends); the call itself allocates and frees nothing.  Inputs whose
 * fluxmi_moe_route_sort_workspace_bytes() exceeds that size are rejected with FLUXMI_ERR_WORKSPACE (the limit
 * is (ceil(ntokens*topk / 512) + 1) * nexperts <= 1048576).  All calls on one GPU share the one array: calls
 * on one stream are ordered, and eager calls issued one after the other from different streams are chained by an
 * event the library keeps per GPU; calls issued at the same moment from several host threads, and replays of a
 * captured graph against other calls, are the caller's to order: they race on the array and give wrong indices.
 * fluxmi_moe_route_sort_static_init() looks up the array's device address for the current device (the only set-up
 * there is); the first call on a device does the same, so a caller whose first call would be under stream capture
 * calls the init function beforehand, outside the capture.  Results are bit-identical to fluxmi_moe_route_sort. */
size_t fluxmi_moe_route_sort_static_max_bytes(void);
int fluxmi_moe_route_sort_static_init(void);
int fluxmi_moe_route_sort_static(const int32_t *choosed, int32_t ntokens, int32_t topk, int32_t nexperts,
                                 int32_t *splits, int32_t *offsets, int32_t *scatter_index,
                                 int32_t *gather_index, int32_t *topk_index, void *stream);

/* Inverse permutation only: `calc_gather_index_impl` (src/moe_ag_scatter/sort_util.cu:121-160).
 * gather_index[scatter_index[i]] = i / topk, topk_index[...] = i % topk for scatter_index[i] in
 * [0, nrows); entries outside are skipped.  topk_index may be NULL. */
int fluxmi_moe_gather_index(const int32_t *scatter_index, int32_t nrows, int32_t topk,
                            int32_t *gather_index, int32_t *topk_index, void *stream);

/* ------------------------------------------------------------------------------------------------
 * Grouped GEMM over ragged per-expert row counts (layer0 and the GEMM half of layer1).
 *
 * Stands in for the kernels behind `GemmGroupedV3AGScatterOp::forward_impl`
 * (src/moe_ag_scatter/ths_op/gemm_grouped_v3_ag_scatter.cc:227-447, arguments
 * include/flux/args/moe_ag_scatter.h:25-35) and the GEMM part of `GemmGroupedV3GatherRS`
 * (src/moe_gather_rs/ths_op/gemm_grouped_v3_gather_rs.cc:245-537, include/flux/args/moe_gather_rs.h:78-117)
 * and the plain `GemmGroupedV3` (src/comm_none/ths_op/gemm_grouped_v3.cc:43-171):
 *
 *   for sorted row r of expert e (offsets[e] <= r < offsets[e+1], offsets = prefix sum of splits):
 *     acc[n]   = sum_k float(A[gather_a ? gather_a[r] : r, k]) * float(B[e, n, k])        (fp32)
 *     D[scatter_d ? scatter_d[r] : r, n] =
 *         bf16( acc[n] * (alpha ? alpha[e] : 1) * (row_scale ? row_scale[r] : 1)
 *                      * (col_scale ? col_scale[e*N + n] : 1) * scalar_scale )
 *
 * A is row-major [*, K] (lda = K), B is [E, N, K] with K contiguous, D is row-major [*, N] in the 16-bit output
 * type of `dtype` (bf16 for bf16 and fp8 operands, fp16 for fp16 operands; "bf16" below stands for that type).
 * `splits` is a DEVICE int32 array of `nexperts` row counts; the tile schedule is derived from it on
 * the device, so the host never reads it.  `max_rows` is an upper bound of sum(splits) (ntokens*topk);
 * rows beyond sum(splits) are not touched.
 *
 * Limits: 1 <= nexperts <= 1024 (FLUXMI_ERR_UNSUPPORTED beyond).  Two kernels stand behind the call.  The
 * MFMA kernel takes every shape with
 *   - rows of K a multiple of 16 bytes: K % 8 == 0 (bf16, fp16), K % 16 == 0 (fp8); a last partial 64-byte step of
 *     K is padded with zeros inside the kernel at full speed;
 *   - N % 4 == 0; a, b 16-byte aligned; d 8-byte (bf16) / 16-byte (fp32) aligned; col_scale 16-byte aligned;
 *   - one expert's weights below 4 GiB (N * K * element size), and with `gather_a`: a_rows > 0 and the whole
 *     of A below 4 GiB (its rows are addressed with 32-bit byte offsets).
 * Any other shape runs a generic kernel (one thread per output element, roughly 100 times slower, meant for
 * correctness only).  fluxmi_grouped_gemm_kernel_kind() tells which of the two a call would take.
 * ---------------------------------------------------------------------------------------------- */
typedef struct fluxmi_grouped_gemm_args {
  int32_t dtype;         /* fluxmi_dtype of A and B */
  int32_t nexperts;      /* E */
  int32_t max_rows;      /* upper bound on the number of sorted rows */
  int32_t n;             /* N, columns of D / rows of each B[e] */
  int32_t k;             /* K */
  int32_t a_rows;        /* rows of A when gather_a is given: entries are clamped into [0, a_rows); 0 = trust them (and take the slow generic kernel: the MFMA kernel needs the extent of a gathered A) */
  const void *a;         /* [rows_a, K] */
  const void *b;         /* [E, N, K] */
  void *d;               /* [max_rows, N] bf16 (fp32 when d_fp32 != 0) */
  const int32_t *splits; /* device [E] */
  const int32_t *gather_a;  /* device [max_rows] or NULL */
  const int32_t *scatter_d; /* device [max_rows] or NULL */
  const float *alpha;       /* device [E] or NULL  (Flux `output_scale` / `weight_scale`) */
  const float *row_scale;   /* device [max_rows] or NULL, indexed by sorted row */
  const float *col_scale;   /* device [E, N] or NULL */
  float scalar_scale;       /* host scalar, 1.0f for none (Flux `input_scale[0]` is passed by pointer below) */
  int32_t d_fp32;           /* 0: D is bf16 (fp16 for FLUXMI_FP16); 1: D is fp32 [max_rows, N] (unrounded layer1 intermediate) */
  const float *scalar_scale_dev; /* device [1] or NULL; multiplied in if given */
  /* Launch tuning; all zero = defaults.  None of them changes a result bit. */
  int32_t cu_margin;     /* compute units left free for other work (Flux `sm_margin`) */
  int32_t raster_rows;   /* row tiles of an expert walked together over all weight panels; 0 = 8 */
  int32_t sched_flags;   /* FLUXMI_SCHED_* */
  int32_t reserved;      /* must be 0 */
} fluxmi_grouped_gemm_args;

#define FLUXMI_SCHED_WHOLE_TAIL_TILES 1 /* do not cut the tiles of the last, partly filled round into pieces */
#define FLUXMI_SCHED_NO_HALF_TILES 2    /* run the last row tile of an expert 256 rows high even if 128 cover it, and the last column tile 256 wide even if 128 cover it */
#define FLUXMI_SCHED_NO_SKINNY_TAIL 4    /* never move the last row tiles of experts that hold at most 64 rows behind all other tiles as 64 x 64 pieces */
#define FLUXMI_SCHED_FORCE_SKINNY_TAIL 8 /* always do so (by default only when those pieces fill at most two rounds of the launch and K spans at least 128 steps of 64 bytes) */
#define FLUXMI_SCHED_HALF_LINE_FILLS 16  /* fill the operand ring of the MFMA kernel with 64-byte half lines, one k-step per ring stage */
#define FLUXMI_SCHED_WHOLE_LINE_FILLS 32 /* fill it with whole 128-byte lines, two k-steps per ring unit (default: only for rows of K of at least 16 KiB that are not gathered; fp16 operands always run the half-line form); not both flags */

size_t fluxmi_grouped_gemm_workspace_bytes(const fluxmi_grouped_gemm_args *args);
int fluxmi_grouped_gemm(const fluxmi_grouped_gemm_args *args, void *workspace,
                        size_t workspace_bytes, void *stream);

/* Which kernel fluxmi_grouped_gemm would run for `args` (nothing is launched): 1 the MFMA kernel, 0 the
 * generic kernel, negative = the fluxmi_status the call itself would return.  The reference has no slow
 * path to report (its TMA kernels take any 16-byte aligned K: gemm_grouped_v3_ag_scatter.cc:249-262 checks
 * shapes only); callers use this to assert they are not on the generic kernel. */
int fluxmi_grouped_gemm_kernel_kind(const fluxmi_grouped_gemm_args *args);

/* ------------------------------------------------------------------------------------------------
 * Top-k reduction fused into the grouped GEMM's epilogue (layer1 in one pass, no [M, N] intermediate):
 *
 *   out[t, n] = bf16( sum over sorted rows r with token_of_row[r] == t of
 *                       acc[r, n] * alpha[e] * row_scale[r] * col_scale[e, n] * scalar_scale )
 *
 * Stands in for the fused GEMM + top-k reduce kernel of `GemmGroupedV3GatherRS`
 * (src/moe_gather_rs/sm90_gemm_array_threadblock_specialized.hpp:1306-1409 reduce, :1916-2086 GEMM).  The
 * epilogue adds each scaled fp32 result into row token_of_row[r] of a fp32 [ntokens, N] workspace with
 * hardware float atomics; a pass before clears the workspace, a pass after rounds it to bf16 `out`.
 * `token_of_row` is the device array gather_index ([max_rows] int32: the token of each sorted row; entries
 * outside [0, ntokens) are skipped).  args->d, d_fp32 and scatter_d are not used (scatter_d must be NULL);
 * every other member means what it means for fluxmi_grouped_gemm.  With top-2 the result does not depend on the
 * order of the additions; with more terms per token the last bits can differ from run to run (fp32 addition is
 * not associative), far inside the 1e-2 bound.  The two-pass form (fluxmi_grouped_gemm with d_fp32 = 1, then
 * fluxmi_topk_gather_reduce) is deterministic for every top-k.
 * ---------------------------------------------------------------------------------------------- */
size_t fluxmi_grouped_gemm_topk_reduce_workspace_bytes(int32_t ntokens, int32_t n);
int fluxmi_grouped_gemm_topk_reduce(const fluxmi_grouped_gemm_args *args, const int32_t *token_of_row,
                                    int32_t ntokens, void *out, void *workspace, size_t workspace_bytes,
                                    void *stream);

/* ------------------------------------------------------------------------------------------------
 * Block-scaled fp8 grouped GEMM (DeepSeek-style 1 x 128 activation scales, 128 x 128 weight scales):
 *
 *   acc[r, n] = sum over scale blocks kb of K ( a_scale[row, kb] * b_scale[e, n / 128, kb] *
 *                 sum_{k in block kb} float(A[row, k]) * float(B[e, n, k]) ),   row = gather_a ? gather_a[r] : r
 *   D as for fluxmi_grouped_gemm (alpha, row_scale, col_scale, scalar scales, scatter_d, d_fp32 all apply).
 *
 * Stands in for the kernels behind `BlockScaleGemm::forward_grouped` / `forward`
 * (src/comm_none/ths_op/blockscale_gemm.cc:648-782, arguments include/flux/args/comm_none.h:169-184; reference
 * semantics test/python/gemm_only/test_blockwise_scale_gemm_only.py:200-262): the products of each 128 of K are
 * summed exactly in fp32 and promoted into the result with their scales.  dtype must be FLUXMI_FP8_E4M3 and
 * K % 128 == 0.  Scale layouts (both are the `scale_inv` outputs of the quantisation entry points below or the
 * reference's own operand layouts):
 *   a_scale  FLUXMI_ASCALE_BLOCK128: [ceil(rows_a / 128), K / 128, 128], the row inside its block of 128 rows
 *            fastest — what fluxmi_quant_e4m3_block128 / quantize_vector_blockwise write for the A matrix
 *            (indexed by the row of A that is read, so it works with gather_a);
 *            FLUXMI_ASCALE_EXPERT_K_M: experts back to back, each [K / 128, rows of the expert] (rows fastest),
 *            expert e starting at float offset offsets[e] * K / 128 — what forward_grouped takes
 *            (blockscale_gemm.cc:717-718); not with gather_a.
 *   b_scale  FLUXMI_BSCALE_N_K: [E, ceil(N / 128), K / 128] — what fluxmi_quant_e4m3_square writes for B;
 *            FLUXMI_BSCALE_K_N: [E, K / 128, ceil(N / 128)] — what forward_grouped takes (:719-721).
 * ---------------------------------------------------------------------------------------------- */
#define FLUXMI_ASCALE_BLOCK128 0
#define FLUXMI_ASCALE_EXPERT_K_M 1
#define FLUXMI_BSCALE_N_K 0
#define FLUXMI_BSCALE_K_N 1
#define FLUXMI_BSCALE_COL_N_K 2 /* one scale per column of B and 128 of K: [E, ceil(N / 128), K / 128, 128], column
                                   inside its block fastest (the `is_groupwise_b` form of BlockScaleGemm::reference,
                                   src/comm_none/ths_op/blockscale_gemm.cc:954-973); served by the generic kernel */
int fluxmi_grouped_gemm_blockscale(const fluxmi_grouped_gemm_args *args, const float *a_scale,
                                   int32_t a_scale_layout, const float *b_scale, int32_t b_scale_layout,
                                   void *stream);

/* The same rows times `ngroups` (1..4) weight tensors in ONE launch, each group with an output of its own:
 * `GemmGroupedV3AGScatterOp::forward_multiple_weights` (gate and up projections sharing the gathered
 * A tiles; src/moe_ag_scatter/ths_op/gemm_grouped_v3_ag_scatter.cc:375-395).  b, d and alpha are
 * HOST arrays of `ngroups` device pointers (alpha itself, or single entries of it, may be NULL); the b, d
 * and alpha members of `args` are ignored, every other member is shared by all groups.  The column tiles
 * of all groups form one tile schedule, so the tail of the launch is shared as well. */
int fluxmi_grouped_gemm_multi(const fluxmi_grouped_gemm_args *args, int32_t ngroups, const void *const *b,
                              void *const *d, const float *const *alpha, void *workspace,
                              size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------------
 * Top-k (weighted) gather-reduce back to token order (the reduce half of layer1).
 *
 * Stands in for `topk_reduce_scatter_impl` behind `flux.topk_scatter_reduce`
 * (src/moe_gather_rs/moe_utils.cu:282-395, src/moe_gather_rs/ths_op/topk_scatter_reduce.cc:30-56), the
 * reduce part of the fused layer1 kernel (src/moe_gather_rs/sm90_gemm_array_threadblock_specialized.hpp:1306-1409)
 * and its weighted form (src/moe_gather_rs/topk_gather_rs_v2.cu:394-407):
 *
 *   out[t, n] = bf16( scale * sum_{g < ngroups} sum_{j < topk}
 *                       w[r] * float(in[g][r, n]) ),   r = routing_idx[t*topk + j],
 *   w[r] = row_weight ? row_weight[r] : 1;  fp32 accumulation in the order g-major then j; one rounding at
 *   the end.
 * `in` is an array (on the HOST) of `ngroups` device pointers to row-major [ntokens*topk, n] matrices.
 * `io_format` names the element types: 0 bf16 in, bf16 out; 1 fp32 in (the unrounded intermediate of
 * fluxmi_grouped_gemm with d_fp32 = 1), bf16 out; 2 fp16 in, fp16 out; 3 fp32 in, fp16 out.  Entries of
 * routing_idx outside [0, ntokens*topk) name no row: they are skipped (negative = a dropped pair) and never
 * dereferenced.
 * Requirements: n % 8 == 0, 1 <= ngroups <= 4, 1 <= topk <= 64.
 * ---------------------------------------------------------------------------------------------- */
int fluxmi_topk_gather_reduce(const void *const *in, int32_t ngroups, int32_t io_format,
                              const int32_t *routing_idx, const float *row_weight, float scale,
                              int32_t ntokens, int32_t topk, int32_t n, void *out, void *stream);

/* ------------------------------------------------------------------------------------------------
 * bf16 -> fp8-e4m3 absmax quantisation, one scale per (row, block of `block_cols` columns).
 *
 * Stands in for `block_scaled_1d_cast_transpose_impl` behind `Quantization::quantize_vector_blockwise`
 * (src/quantization/quantization.cu:306-367, :421-706, :1382-1456; src/quantization/ths_op/quantization.cc:75-145):
 *   amax  = max |float(x)| over the block,  a = max(amax, eps)
 *   scale = 1 if a == 0; 448 / a (fp32 division); if that is +inf, 0x1.FEp127
 *   q     = e4m3_round_nearest_even_saturate( float(x) * scale )
 *   scale_inv = float(1.0 / double(scale))
 * block_cols == 0 means one block per row (per-token scale, scale_inv is [rows]); block_cols == 128 is
 * Flux's 1x128 form.  With `permute_scale` != 0 and block_cols == 128 scale_inv is stored as
 * [ceil(rows/128), ceil(cols/128), 128] (row-in-block fastest), otherwise as [rows, nblocks].
 * Requirements: cols % 8 == 0.
 * ---------------------------------------------------------------------------------------------- */
int fluxmi_quant_e4m3_rowwise(const void *x_bf16, int64_t rows, int64_t cols, int32_t block_cols,
                              float eps, void *q_out, float *scale_inv_out, int32_t permute_scale,
                              void *stream);

/* ------------------------------------------------------------------------------------------------
 * bf16 -> fp8-e4m3 absmax quantisation with one scale per 128 x 128 block of each [rows, cols] matrix of
 * a batch, and optionally a transposed copy of the bytes.
 *
 * Stands in for `block_scaled_cast_transpose_impl` behind `Quantization::quantize_square_blockwise`
 * (batch = 1) and `Quantization::batch_quantize_square_blockwise` (src/quantization/quantization.cu:1185-1380
 * full blocks, :971-1183 ragged blocks, :1458-1528 dispatch; src/quantization/ths_op/quantization.cc:152-316):
 *   amax, scale, q as for fluxmi_quant_e4m3_rowwise, taken over the part of the block inside the matrix;
 *   scale_inv = 1.0f / scale (fp32 division).
 * x is [batch, rows, cols] bf16; q_out [batch, rows, cols] bytes; scale_inv_out
 * [batch, ceil(rows/128), ceil(cols/128)].  With q_t_out / scale_inv_t_out (both or neither):
 * q_t_out[b, c, r] = q_out[b, r, c] and scale_inv_t_out [batch, ceil(cols/128), ceil(rows/128)] holds the
 * same scales transposed.  Any rows / cols; 16-byte accesses are used when cols % 8 == 0 (and, for the
 * transposed copy, rows % 16 == 0) and the pointers are aligned accordingly.
 * ---------------------------------------------------------------------------------------------- */
int fluxmi_quant_e4m3_square(const void *x_bf16, int64_t batch, int64_t rows, int64_t cols, float eps,
                             void *q_out, float *scale_inv_out, void *q_t_out, float *scale_inv_t_out,
                             void *stream);

/* ------------------------------------------------------------------------------------------------
 * bf16 -> fp8-e4m3 absmax quantisation with one scale per (row, 128-column block) and, optionally, the
 * transposed matrix quantised with one scale per (column, 128-row block), from a single read of x.
 *
 * Stands in for `block_scaled_1d_cast_transpose_impl` behind `Quantization::quantize_vector_blockwise`
 * including its `return_transpose` outputs (src/quantization/quantization.cu:421-706 ragged, :708-969 full
 * blocks, :1382-1456 dispatch; src/quantization/ths_op/quantization.cc:75-145).  Arithmetic as for
 * fluxmi_quant_e4m3_rowwise (scale_inv = float(1.0 / double(scale))); what lies outside the matrix counts as 0.
 *   q_out [rows, cols], scale_inv_out [ceil(rows/128), ceil(cols/128), 128] (row inside its block fastest;
 *   entries of rows past the end are not written);
 *   q_t_out [cols, rows], scale_inv_t_out [ceil(cols/128), ceil(rows/128), 128] (both or neither):
 *   q_t_out[c, r] = e4m3(x[r, c] * scale_t(c, r / 128)).
 * Any rows / cols; 16-byte accesses when cols % 8 == 0 (transposed: rows % 16 == 0) and aligned pointers.
 * ---------------------------------------------------------------------------------------------- */
int fluxmi_quant_e4m3_block128(const void *x_bf16, int64_t rows, int64_t cols, float eps, void *q_out,
                               float *scale_inv_out, void *q_t_out, float *scale_inv_t_out, void *stream);

/* ------------------------------------------------------------------------------------------------
 * Calibration streams (no counterpart in the reference; for benchmarks): what the memory system of the GPU at
 * hand gives a kernel that only streams.  copy == 0: every byte of src[0, bytes) is read once (16 bytes per lane
 * and load, eight loads in flight per lane) and fluxmi_calib_stream_sink_bytes() bytes of dst are written;
 * copy != 0: the same reads, each stored to dst[0, bytes).  bytes and both pointers are multiples of 16.
 * ---------------------------------------------------------------------------------------------- */
size_t fluxmi_calib_stream_sink_bytes(void);
int fluxmi_calib_stream(const void *src, void *dst, size_t bytes, int32_t copy, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLUXMI_H_ */
