/*
 * C ABI of libflexshard_hip.so: hand-written gfx950 (MI355X) kernels for the
 * single-GPU hot path of FlexShard's bucketed placements.
 *
 * The reference has no FFI: its hot path is Python calling Triton kernels, one
 * third-party Triton quantizer and ATen ops.  Each entry point below replaces
 * the device work of the reference lines it cites (paths under the reference
 * checkout, src/flex_shard/...).  The Python placements in flex_shard_amd/
 * are the only callers.
 *
 * Conventions
 *  - every function returns 0 on success and a negative FSH_E* code otherwise;
 *    fsh_last_error() returns a thread-local message for the last failure;
 *  - nothing here allocates or frees device memory, synchronizes the host, or
 *    touches the null stream: `stream` is a hipStream_t passed as void*, and
 *    all work is queued on it;
 *  - pointers named *_dev are device pointers; plain struct tables are host
 *    memory read during the call;
 *  - sizes and offsets are int64_t; offsets are in bytes unless the name says
 *    otherwise.
 */
#ifndef FLEXSHARD_HIP_H_
#define FLEXSHARD_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSH_OK 0
#define FSH_EINVAL (-22)  /* bad argument, message in fsh_last_error() */
#define FSH_ENOTSUP (-95) /* valid request this build cannot serve */
#define FSH_EHIP (-5)     /* a HIP runtime call failed */

/* Library version, (major << 16) | minor. */
int32_t fsh_version(void);
/* Message of the calling thread's last failed call ("" if none). */
const char* fsh_last_error(void);

/* ------------------------------------------------------------------------
 * 1. Fused tile quantize + pack.
 * Replaces custom_placements/blockwise_quant_bucketed_block_shard.py:792-897
 * (_pack_local_quantized_chunks: pad zeroing, dtype staging, one quantizer
 * launch per chunk, two foreach copies) and the quantizer it calls,
 * custom_placements/fp8_bucketed_block_shard.py:66-88.  Arithmetic per
 * block x block tile follows tests/test_flex_shard_fp8_allgather.py:45-90:
 *   amax in the quantization dtype, floor 1e-12, scale = fp32(448 / fp64(amax)),
 *   q = e4m3fn(fp32(x) * scale), stored scale = 1.0f / scale.
 * One launch covers every chunk of a rank and zeroes the payload's two pad
 * gaps.
 * ---------------------------------------------------------------------- */

/* Source element kinds. */
#define FSH_SRC_BF16 0        /* bf16 shard, quantized as is                  */
#define FSH_SRC_F32 1         /* fp32 shard, quantized as fp32                */
#define FSH_SRC_F32_AS_BF16 2 /* fp32 master shard, rounded to bf16 first     */
#define FSH_SRC_F16 3         /* fp16 shard, quantized as is                  */
#define FSH_SRC_F32_AS_F16 4  /* fp32 master shard, rounded to fp16 first     */

/* Floor applied to a tile's amax. */
#define FSH_EPS_INPUT_DTYPE 0 /* 1e-12 rounded to the quantization dtype      */
#define FSH_EPS_FP32 1        /* 1e-12 rounded to fp32 whatever the dtype     */

typedef struct fsh_quant_chunk {
  const void* src_dev;    /* first element of the chunk's [rows, in_dim] matrix */
  int64_t rows;           /* > 0 */
  int64_t in_dim;         /* > 0 */
  int64_t src_row_stride; /* elements between consecutive rows, >= in_dim      */
  int64_t qdata_offset;   /* byte offset of the chunk's FP8 bytes in payload   */
  int64_t scale_offset;   /* byte offset of its fp32 scale block, 4-aligned    */
  int32_t src_kind;       /* FSH_SRC_*                                        */
  int32_t reserved;
} fsh_quant_chunk;

#define FSH_MAX_QUANT_CHUNKS 24

/*
 * payload_dev[qdata_offset + r*in_dim + c] = FP8 byte of element (r, c);
 * scales of tile (tr, tc) at scale_offset + 4*(tr*ceil(in_dim/block) + tc).
 * Bytes [zero0_begin, zero0_end) and [zero1_begin, zero1_end) of the payload
 * are set to zero (the pad between data and scales, and the tail pad).
 * nchunks <= FSH_MAX_QUANT_CHUNKS; block = 128 takes the vectorized path when
 * a chunk's pointers, stride and offsets are 16-byte friendly, any other
 * block size or alignment takes a scalar path with the same results.
 */
int fsh_quantize_pack(const fsh_quant_chunk* chunks, int32_t nchunks, void* payload_dev,
                      int64_t payload_nbytes, int64_t zero0_begin, int64_t zero0_end,
                      int64_t zero1_begin, int64_t zero1_end, int32_t block, int32_t eps_mode,
                      void* stream);

/*
 * The same launch as a reusable plan, for a bucket whose shards stay where
 * they are from step to step (sharded parameter storage is persistent):
 * everything but the payload address and the stream is checked and stored
 * once, and a steady-state pack is one call with three arguments.  Serves the
 * per-step repetition of _pack_local_quantized_chunks
 * (custom_placements/blockwise_quant_bucketed_block_shard.py:792-897), which
 * the reference re-derives in Python on every unshard.  Any number of chunks:
 * more than FSH_MAX_QUANT_CHUNKS become several launches inside one call, the
 * first of which zeroes the pad ranges.  The plan holds the chunks' source
 * addresses: the caller launches it only while the same memory is behind
 * them.  A plan is host memory only (no device allocation); launches of one
 * plan may be issued from several threads and streams at once.
 */
int fsh_quant_pack_plan_create(const fsh_quant_chunk* chunks, int32_t nchunks, int64_t payload_nbytes,
                               int64_t zero0_begin, int64_t zero0_end, int64_t zero1_begin,
                               int64_t zero1_end, int32_t block, int32_t eps_mode, void** plan_out);
/* payload_dev: payload_nbytes bytes, 16-byte aligned. */
int fsh_quant_pack_plan_launch(const void* plan, void* payload_dev, void* stream);
void fsh_quant_pack_plan_destroy(void* plan);

/* ------------------------------------------------------------------------
 * 2. Segment copy / zero / cast-pack.
 * Replaces the Triton kernels of custom_placements/_copy_kernels.py:
 * _copy_segments_kernel (:123-142, launcher :436-461), _zero_segments_kernel
 * (:145-161, :464-484) and the four _pack_segments_* kernels (:17-120,
 * :249-359).  The three int64 device arrays are the same arrays the Triton
 * kernels take, in units of `unit_nbytes` (1, 2, 4, 8 or 16).
 * ---------------------------------------------------------------------- */
int fsh_copy_segments(const void* src_dev, void* dst_dev, const int64_t* src_offsets_dev,
                      const int64_t* numels_dev, const int64_t* dst_offsets_dev,
                      int64_t nsegments, int64_t max_segment_numel, int32_t unit_nbytes,
                      void* stream);

int fsh_zero_segments(void* dst_dev, const int64_t* numels_dev, const int64_t* dst_offsets_dev,
                      int64_t nsegments, int64_t max_segment_numel, int32_t unit_nbytes,
                      void* stream);

#define FSH_DT_BF16 0
#define FSH_DT_F32 1
#define FSH_DT_F16 2 /* fsh_unpack_dequant's dequantized output only */
/* out[dst_off[s]+i] = cast(inputs[tensor_idx[s]][src_off[s]+i]), i < numel[s];
 * offsets in elements; input_ptrs_dev holds the inputs' device addresses.  A
 * negative tensor index makes the segment a zero fill, so one launch can
 * build a whole zero-padded send buffer. */
int fsh_pack_segments(const int64_t* input_ptrs_dev, const int64_t* tensor_indices_dev,
                      const int64_t* src_offsets_dev, const int64_t* numels_dev,
                      const int64_t* dst_offsets_dev, int64_t nsegments,
                      int64_t max_segment_numel, int32_t src_dtype, int32_t dst_dtype,
                      void* dst_dev, void* stream);

/* ------------------------------------------------------------------------
 * 3. Unpack of gathered rank rows: compaction fused with bf16 dequantization.
 * Replaces custom_placements/blockwise_quant_bucketed_block_shard.py:1237-1422
 * (_finish_quant_unshard_from_rank_rows / _copy_out_rank_rows_triton) and
 * blockwise_fp8/blockwise_fp8_weight.py:25-54,121-127 (blockwise_dequant_weight)
 * in one pass over the FP8 bytes.
 * ---------------------------------------------------------------------- */
typedef struct fsh_unpack_chunk {
  int64_t src_qdata_offset;   /* bytes from rows_dev to the chunk's FP8 rows    */
  int64_t src_scale_offset;   /* bytes from rows_dev to its fp32 scale block    */
  int64_t rows;
  int64_t in_dim;
  int64_t dst_qdata_offset;   /* bytes into compact_dev                         */
  int64_t dst_scale_offset;   /* bytes into compact_dev                         */
  int64_t dst_dequant_offset; /* elements into dequant_dev                      */
} fsh_unpack_chunk;

/*
 * chunks_dev: device table of nchunks entries; total_tiles = sum over chunks
 * of ceil(rows/block)*ceil(in_dim/block); tile_starts_dev[i] = first tile
 * index of chunk i (nchunks+1 entries, exclusive prefix sum).
 * compact_dev may be NULL (no compaction), dequant_dev may be NULL (no
 * dequantization).  dequant dtype is FSH_DT_BF16, FSH_DT_F32 or FSH_DT_F16.
 */
int fsh_unpack_dequant(const void* rows_dev, const fsh_unpack_chunk* chunks_dev,
                       const int64_t* tile_starts_dev, int32_t nchunks, int64_t total_tiles,
                       void* compact_dev, void* dequant_dev, int32_t dequant_dtype,
                       int32_t block, void* stream);

/* ------------------------------------------------------------------------
 * 4. fp32 gradient accumulation of one microbatch.
 * Replaces the AccumulateGrad cast-and-add the runtime relies on
 * (flex_shard/bucket_runtime.py:931-933, policy flex_shard/bucket_storage.py
 * :59-77): acc[i] = acc[i] + float(grad[i]); with overwrite != 0,
 * acc[i] = float(grad[i]) (first microbatch).
 * ---------------------------------------------------------------------- */
int fsh_accumulate_grad(float* acc_dev, const void* grad_dev, int32_t grad_dtype, int64_t numel,
                        int32_t overwrite, void* stream);

/* ------------------------------------------------------------------------
 * 5. Fixed-order W-way reduction of one rank's range (single-GPU stand-in
 * for the reduce-scatter).  Replaces custom_placements/utils.py:157-172
 * (reduce_scatter_grads) with the op/divide choices of :116-144, and feeds
 * the copy-out views of custom_placements/block_shard.py:1373-1380.
 *   out[i] = fold over r = 0..world-1, in that order, of
 *            src[r*contribution_stride + column_offset + i]
 * ---------------------------------------------------------------------- */
#define FSH_REDUCE_SUM 0     /* plain sum                                      */
#define FSH_REDUCE_PREMUL 1  /* each term multiplied by `factor` before adding */
#define FSH_REDUCE_POSTMUL 2 /* sum multiplied by `factor`                     */
#define FSH_REDUCE_POSTDIV 3 /* sum divided by `factor`                        */
int fsh_reduce_rows_f32(float* out_dev, const float* src_dev, int64_t contribution_stride,
                        int32_t world, int64_t column_offset, int64_t numel, int32_t mode,
                        float factor, void* stream);
/* The same fold over bf16 contributions into a bf16 range: terms widened to
 * fp32 (pre-multiplied if asked), added in fp32 in rank order, one rounding to
 * bf16 at the end.  (A ring reduce-scatter in bf16 rounds after every hop; this
 * stand-in does not imitate that.) */
int fsh_reduce_rows_bf16(void* out_dev, const void* src_dev, int64_t contribution_stride, int32_t world,
                         int64_t column_offset, int64_t numel, int32_t mode, float factor, void* stream);

/* ------------------------------------------------------------------------
 * 6. Newton-Schulz orthogonalization on MFMA.
 * Replaces dist_muon/optimizer.py:2120-2151 (_zeropower_via_newtonschulz):
 * bf16 operands, fp32 accumulation, every product rounded to bf16.
 * x_dev: batch matrices [rows, cols] bf16, row-major, batch stride rows*cols,
 * overwritten with the result.  Tall matrices (rows > cols) are iterated in
 * place through X <- a X + X (b A + c A A), A = X^T X, which is the transpose
 * of the reference's iteration on X^T.
 * workspace_dev: at least fsh_newton_schulz_workspace_bytes(...) bytes.
 * ---------------------------------------------------------------------- */
int64_t fsh_newton_schulz_workspace_bytes(int64_t batch, int64_t rows, int64_t cols);
int fsh_newton_schulz(void* x_dev, int64_t batch, int64_t rows, int64_t cols, float a, float b,
                      float c, int32_t steps, float eps, void* workspace_dev,
                      int64_t workspace_nbytes, void* stream);

/* Several batches of different shapes in one call (the per-shape groups of
 * the owned matrices of dist_muon/optimizer.py, which the reference runs one
 * after the other through :2120-2151).  Results are identical to calling
 * fsh_newton_schulz once per problem; the same product of all problems is
 * issued together so that the short tiles of one shape fill the last,
 * partly empty round of workgroups of another.  Problems must not overlap. */
typedef struct fsh_ns_problem {
  void* x_dev;             /* [batch, rows, cols] bf16, overwritten            */
  int64_t batch, rows, cols;
  void* workspace_dev;     /* >= fsh_newton_schulz_workspace_bytes(batch, rows, cols) */
  int64_t workspace_nbytes;
} fsh_ns_problem;
#define FSH_MAX_NS_PROBLEMS 16
int fsh_newton_schulz_multi(const fsh_ns_problem* problems, int32_t count, float a, float b, float c,
                            int32_t steps, float eps, void* stream);

/* Allocation-free variant of fsh_newton_schulz.  It has no counterpart in the
 * reference: it is for callers that cannot allocate device memory or bring a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  The workspace is a static device array of
 * FSH_NS_STATIC_SCRATCH_BYTES inside the library, held on every GPU the
 * library runs on until the process ends; its address on the current device
 * is resolved on the first call on that device (so make that first call
 * outside any graph capture).  The call allocates and frees nothing.  A batch
 * whose fsh_newton_schulz_workspace_bytes() exceeds the static scratch is
 * rejected with FSH_ENOTSUP.  All calls on one GPU share the one array: calls
 * that overlap on a GPU (different streams, or threads) race and must be
 * serialized by the caller; calls on one stream are ordered by the stream.
 * Results are those of fsh_newton_schulz, bit for bit. */
#define FSH_NS_STATIC_SCRATCH_BYTES (128LL << 20)
int fsh_newton_schulz_noalloc(void* x_dev, int64_t batch, int64_t rows, int64_t cols, float a, float b,
                              float c, int32_t steps, float eps, void* stream);

/* Batched bf16 "NT" GEMM, the building block of (6), exported for tests:
 *   C[b] = bf16(alpha * A[b] . B[b]^T + beta * D[b] + diag_add * I)   fp32 accumulation
 * A is [m, k] with row stride lda, B is [n, k] with row stride ldb (both
 * k-contiguous; see k_major for the other layout), D and C are [m, n] with
 * row strides ldd / ldc.  D may be NULL
 * (beta ignored) or alias C.  ct_dev, when not NULL, also receives C[b]^T as
 * an [n, m] matrix with row stride ldct.  Batch strides are in elements.
 * k and all leading dimensions must be multiples of 8 and all pointers
 * 16-byte aligned; m and n are arbitrary. */
typedef struct fsh_gemm_desc {
  const void* a_dev;
  const void* b_dev;
  const void* d_dev;
  void* c_dev;
  void* ct_dev;
  int64_t m, n, k;
  int64_t lda, ldb, ldd, ldc, ldct;
  int64_t batch;
  int64_t stride_a, stride_b, stride_d, stride_c, stride_ct;
  float alpha, beta;
  int32_t symmetric; /* nonzero: the caller guarantees a symmetric result (m == n, e.g. b == a
                        and d symmetric); only the tiles on or above the diagonal are
                        computed and the rest is mirrored.  ct_dev must be null. */
  float diag_add;    /* added to C[b][i][i] in fp32 before the rounding to bf16 (0: plain product) */
  int32_t k_major;   /* nonzero: A is [k, m] and B is [k, n] (row strides lda / ldb), so the product
                        is A^T . B; same products in the same order as the k-contiguous form on
                        the transposed operands.  Needs m, n multiples of 256, k of 64, and at
                        least 192 tiles of 256 x 256 in all. */
  int32_t reserved;  /* zero */
} fsh_gemm_desc;
int fsh_gemm_bf16_nt(const fsh_gemm_desc* desc, void* stream);
/* `count` independent products; those that qualify for the large-tile kernel
 * share launches.  Same results as `count` calls of fsh_gemm_bf16_nt. */
int fsh_gemm_bf16_nt_group(const fsh_gemm_desc* descs, int32_t count, void* stream);

/* ------------------------------------------------------------------------
 * 7. Muon elementwise steps in bf16 (fp32 math, one rounding per reference
 * tensor op).  Replace dist_muon/optimizer.py:2049-2068 (_prepare_muon_input:
 * momentum.lerp_(grad, 1-mu); out = lerp(grad, momentum, mu) when nesterov)
 * and :2100-2117 (_apply_muon_update: p *= 1 - lr*wd; p += -adjusted_lr*dir).
 * ---------------------------------------------------------------------- */
int fsh_muon_prepare(void* momentum_dev, const void* grad_dev, void* out_dev, int64_t numel,
                     float lerp_weight /* 1 - mu */, float nesterov_weight /* mu */,
                     int32_t nesterov, void* stream);
int fsh_muon_apply(void* param_dev, const void* direction_dev, int64_t numel, float decay_factor,
                   float neg_adjusted_lr, float direction_scale, void* stream);
/* The same two steps of the same reference lines on fp32 master state (fp32
 * gradient, momentum buffer and parameter, as the reference's own optimizer
 * tests use): the momentum and the parameter are updated in fp32 with no
 * intermediate rounding; `out` is the bf16 input of the orthogonalization
 * (the cast of dist_muon/optimizer.py:2131), `direction` its bf16 result,
 * scaled in fp32 when direction_scale != 1 (:2093-2096 on an fp32 buffer). */
int fsh_muon_prepare_f32(float* momentum_dev, const float* grad_dev, void* out_bf16_dev, int64_t numel,
                         float lerp_weight, float nesterov_weight, int32_t nesterov, void* stream);
int fsh_muon_apply_f32(float* param_dev, const void* direction_bf16_dev, int64_t numel, float decay_factor,
                       float neg_adjusted_lr, float direction_scale, void* stream);

/* ------------------------------------------------------------------------
 * 8. Forward product of a linear layer with a prequantized weight.
 * Replaces the device work of blockwise_fp8/fp8_blockwise_linear.py:50-91
 * (Fp8BlockwiseGemms.forward): the activation quantizer and the scaled FP8
 * GEMM it takes from torchao (triton_fp8_blockwise_act_quant_lhs and
 * triton_fp8_gemm_1x128_128x128 of torchao.prototype.blockwise_fp8_training,
 * torchao >= 0.18, not vendored by the reference).
 *
 * fsh_act_quant_1x128: x is [rows, cols] bf16 with row stride ldx.  Every
 * run of 128 consecutive elements of a row (the last one zero-padded) is
 * quantized like a weight tile: amax floored at 1e-12, scale = fp32(448 /
 * fp64(amax)), q = e4m3fn(fp32(x) * scale).  q_dev is [rows, ldq] bytes with
 * ldq = cols rounded up to 128 (pad bytes are written as zero), scales_dev is
 * the [ldq / 128, rows] table of 1.0f / scale (row index contiguous).
 *
 * fsh_fp8_gemm_1x128_128x128:
 *   out[i][j] = bf16( sum over kb of dot(xq[i][kb], wq[j][kb])
 *                                  * (xs[kb][i] * ws[j / 128][kb]) ),  fp32 sums,
 * xq [m, k] and wq [n, k] E4M3FN bytes with row strides ldxq / ldwq, xs the
 * [k / 128, m] table above, ws the weight's [ceil(n / 128), ws_cols] scales,
 * out [m, n] bf16 with row stride ldo.  k must be a multiple of 128.
 * ---------------------------------------------------------------------- */
int fsh_act_quant_1x128(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_dev,
                        int64_t ldq, float* scales_dev, int32_t eps_mode, void* stream);
int fsh_fp8_gemm_1x128_128x128(const void* xq_dev, const float* xs_dev, const void* wq_dev,
                               const float* ws_dev, void* out_dev, int64_t m, int64_t n, int64_t k,
                               int64_t ldxq, int64_t ldwq, int64_t ldo, int64_t ws_cols, void* stream);

/* ------------------------------------------------------------------------
 * 9. Backward products of the same linear layer.  Replace the device work of
 * blockwise_fp8/fp8_blockwise_linear.py:93-162 (Fp8BlockwiseGemms.backward):
 *
 * input gradient (:107-126)   grad_x = grad_out . W: fsh_act_quant_1x128 on
 *   grad_out (runs along the output index), fsh_fp8_transpose of the weight
 *   bytes (replaces _as_column_major_2d at :113; the scales are read across,
 *   no copy), fsh_fp8_gemm_1x128_128x128_dgrad.
 * weight gradient (:127-161)  grad_w = grad_out^T . x: both operands through
 *   fsh_act_quant_128x1_transposed (replaces torchao's
 *   triton_fp8_blockwise_act_quant_transposed_lhs at :134 and
 *   triton_fp8_blockwise_act_quant_rhs at :139; runs of 128 tokens), then
 *   fsh_fp8_gemm_1x128_128x1 (replaces triton_fp8_gemm_1x128_128x1 at :144).
 *
 * fsh_fp8_transpose: dst[c][r] = src[r][c] for a [rows, cols] byte matrix;
 * dst is [cols, ld_dst] with rows <= ld_dst <= rows rounded up to 128, the
 * columns from `rows` on written as zero.
 *
 * fsh_act_quant_128x1_transposed: x is [rows, cols] bf16 with row stride ldx.
 * Every run of 128 consecutive rows of a column (the last run zero-padded) is
 * quantized like a weight tile (see section 8).  q_dev is [cols, ldq] bytes,
 * q[c][r], ldq = rows rounded up to 128 with the pad written as zero;
 * scales_dev is the [ldq / 128, cols] table of 1.0f / scale.
 *
 * fsh_act_quant_both: the output gradient is needed in both forms (runs along
 * the output index for the input gradient, :107-110; runs of 128 tokens,
 * transposed, for the weight gradient, :134-138).  One pass over x writes what
 * fsh_act_quant_1x128 (q_row_dev [rows, ldq_row], scales_row_dev
 * [ldq_row / 128, rows]; ldq_row = cols rounded up to 128) and
 * fsh_act_quant_128x1_transposed (q_col_dev [cols, ldq_col], scales_col_dev
 * [ldq_col / 128, cols]; ldq_col = rows rounded up to 128) would write, bit
 * for bit, reading x once instead of twice.
 *
 * fsh_fp8_gemm_1x128_128x128_dgrad:
 *   out[i][j] = bf16( sum over ob of dot(gq[i][ob], wtq[j][ob])
 *                                  * (gs[ob][i] * ws[ob][j / 128]) ),
 * gq [m, out_dim] and its [out_dim / 128, m] scales from fsh_act_quant_1x128,
 * wtq [in_dim, out_dim] the transposed weight bytes, ws the weight's own
 * [out_dim / 128, ws_cols] table, out [m, in_dim] bf16.  out_dim (the
 * contraction length) must be a multiple of 128.
 *
 * fsh_fp8_gemm_1x128_128x1:
 *   out[i][j] = bf16( sum over kb of dot(aq[i][kb], bq[j][kb])
 *                                  * (as[kb][i] * bs[kb][j]) ),
 * aq [m, k], bq [n, k] bytes and their [k / 128, m] and [k / 128, n] tables
 * (both as fsh_act_quant_128x1_transposed writes them), out [m, n] bf16.
 * ---------------------------------------------------------------------- */
int fsh_fp8_transpose(const void* src_dev, int64_t rows, int64_t cols, int64_t ld_src, void* dst_dev,
                      int64_t ld_dst, void* stream);
int fsh_act_quant_128x1_transposed(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_dev,
                                   int64_t ldq, float* scales_dev, int32_t eps_mode, void* stream);
int fsh_act_quant_both(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_row_dev,
                       int64_t ldq_row, float* scales_row_dev, void* q_col_dev, int64_t ldq_col,
                       float* scales_col_dev, int32_t eps_mode, void* stream);
int fsh_fp8_gemm_1x128_128x128_dgrad(const void* gq_dev, const float* gs_dev, const void* wtq_dev,
                                     const float* ws_dev, void* out_dev, int64_t m, int64_t in_dim,
                                     int64_t out_dim, int64_t ldgq, int64_t ldwt, int64_t ldo,
                                     int64_t ws_cols, void* stream);
int fsh_fp8_gemm_1x128_128x1(const void* aq_dev, const float* as_dev, const void* bq_dev,
                             const float* bs_dev, void* out_dev, int64_t m, int64_t n, int64_t k,
                             int64_t ldaq, int64_t ldbq, int64_t ldo, void* stream);

/* ------------------------------------------------------------------------
 * 10. One whole Muon step over matrices grouped by shape, for an owner's whole
 * parameters (the comm-free step of dist_muon/_optimizer_reshard_runtime.py
 * :645-661): dist_muon/optimizer.py:2049-2068 (momentum, Nesterov), :2120-2151
 * (Newton-Schulz) and :2100-2117 (decayed update), i.e. fsh_muon_prepare,
 * fsh_newton_schulz_multi and fsh_muon_apply in sequence, with the same
 * results bit for bit.  Per group there is one momentum launch for all its
 * matrices (it also leaves the sums of squares the normalization needs, so
 * the Newton-Schulz input is read once less).  The update of a group whose
 * matrices fill the large-tile GEMM kernel is applied by the epilogue of its
 * last Newton-Schulz product (the orthogonalized matrix is then never
 * written); other groups get one update launch.
 * The parameters, gradients and momentum buffers of a group are separate
 * allocations, named by device tables of their addresses; each must be a
 * contiguous [rows, cols] matrix of the group's master_dtype at a 16-byte
 * aligned address.  With fp32 masters the momentum buffers and parameters
 * are updated in fp32 (fsh_muon_prepare_f32 / fsh_muon_apply_f32, same bits),
 * only the Newton-Schulz input is rounded to bf16, and the update is always a
 * separate launch.
 * batch_dev is scratch of batch*rows*cols bf16: it holds the momentum
 * output and, for groups updated by a separate launch, the orthogonalized
 * direction afterwards (its contents after the call are otherwise unspecified).
 * Errors: the argument checks (list, groups, sizes, workspaces) come before
 * any launch.  A failure after them (a launch the runtime rejects, a product
 * the GEMM planner cannot place, an LDS reservation refused) leaves the step
 * half done: the momentum buffers have been advanced, no parameter, or only
 * some, updated.  Treat it as fatal for the optimizer state; do not retry
 * the step.
 * ---------------------------------------------------------------------- */
typedef struct fsh_muon_group {
  const int64_t* param_ptrs_dev;    /* [batch] addresses of the parameters, updated in place   */
  const int64_t* grad_ptrs_dev;     /* [batch] addresses of the gradients                      */
  const int64_t* momentum_ptrs_dev; /* [batch] addresses of the momentum buffers, updated      */
  void* batch_dev;                  /* [batch, rows, cols] bf16 scratch                        */
  int64_t batch, rows, cols;        /* rows, cols multiples of 8                               */
  void* workspace_dev;              /* >= fsh_newton_schulz_workspace_bytes(batch, rows, cols) */
  int64_t workspace_nbytes;
  float neg_adjusted_lr;            /* -lr * shape factor of dist_muon/optimizer.py:2031-2046  */
  float direction_scale;            /* 1, or ratio / reference_ratio of :2082-2097             */
  int32_t master_dtype;             /* FSH_DT_BF16 or FSH_DT_F32: parameters, gradients, momentum */
  int32_t reserved;
} fsh_muon_group;
int fsh_muon_step(const fsh_muon_group* groups, int32_t count, float lerp_weight /* 1 - mu */,
                  float nesterov_weight /* mu */, int32_t nesterov, float decay_factor /* 1 - lr*wd */, float a,
                  float b, float c, int32_t steps, float eps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLEXSHARD_HIP_H_ */
