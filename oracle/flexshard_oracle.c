/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement, in plain C, of the arithmetic on FlexShard's single-GPU
 * data-parallel hot path.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this library; the shipped package
 * never does.
 *
 * Every routine names the reference lines it follows (paths under the
 * reference checkout, `src/flex_shard/...`).  The FP8 conversion is written
 * from the OCP E4M3FN definition rather than from torch's bit tricks, so that
 * agreement with torch's own cast (checked exhaustively in the tests) pins it.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, no fast-math).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FSO_EXPORT __attribute__((visibility("default")))

/* ---------------------------------------------------------------- scalars */

static inline float fso_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* float -> bfloat16, round to nearest even; NaN -> 0x7FC0 (torch's c10
 * round_to_nearest_even convention). */
static inline uint16_t fso_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if (isnan(f)) return 0x7FC0;
  uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)((u + bias) >> 16);
}

/* float -> OCP float8 E4M3FN byte, round to nearest even, non-saturating:
 * magnitudes that round past 448 give the NaN encoding (S.1111.111), as
 * torch's Tensor.to(torch.float8_e4m3fn) does.  Written from the format
 * definition: bias 7, 3 mantissa bits, subnormal step 2^-9, no infinities. */
static inline uint8_t fso_f32_to_e4m3fn(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  if (isnan(x)) return (uint8_t)(sign | 0x7F);
  double a = fabs((double)x);
  if (isinf(x)) return (uint8_t)(sign | 0x7F);
  if (a < 0.015625) { /* below the smallest normal 2^-6: fixed step 2^-9 */
    double q = nearbyint(a * 512.0); /* default mode: ties to even */
    return (uint8_t)(sign | (uint8_t)q); /* q == 8 is exactly 0x08 = 2^-6 */
  }
  int e;
  double m = frexp(a, &e); /* a = m * 2^e, m in [0.5, 1) */
  m *= 2.0;
  e -= 1; /* a = m * 2^e, m in [1, 2) */
  double q = nearbyint((m - 1.0) * 8.0);
  if (q == 8.0) {
    q = 0.0;
    e += 1;
  }
  int code = ((e + 7) << 3) | (int)q;
  if (code > 0x7E) code = 0x7F;
  return (uint8_t)(sign | (uint8_t)code);
}

/* OCP E4M3FN byte -> float (exact). */
static inline float fso_e4m3fn_to_f32(uint8_t b) {
  int sign = b >> 7;
  int ex = (b >> 3) & 0xF;
  int man = b & 7;
  double v;
  if (ex == 0xF && man == 7)
    v = NAN;
  else if (ex == 0)
    v = ldexp((double)man, -9);
  else
    v = ldexp(1.0 + man / 8.0, ex - 7);
  return (float)(sign ? -v : v);
}

FSO_EXPORT uint8_t fso_scalar_f32_to_e4m3fn(float x) { return fso_f32_to_e4m3fn(x); }
FSO_EXPORT float fso_scalar_e4m3fn_to_f32(uint8_t b) { return fso_e4m3fn_to_f32(b); }
FSO_EXPORT uint16_t fso_scalar_f32_to_bf16(float x) { return fso_f32_to_bf16(x); }

/* ------------------------------------------------------- tile quantization */

enum { FSO_SRC_BF16 = 0, FSO_SRC_F32 = 1, FSO_SRC_F32_AS_BF16 = 2 };
enum { FSO_EPS_INPUT_DTYPE = 0, FSO_EPS_FP32 = 1 };

/* The value the quantizer sees for element (r, c): the source dtype itself,
 * or an fp32 master value first rounded to bf16 (the reference stages that
 * cast before quantizing: custom_placements/
 * blockwise_quant_bucketed_block_shard.py:839-853). */
static inline float fso_load(const void *src, int src_kind, int64_t idx) {
  if (src_kind == FSO_SRC_BF16) return fso_bf16_to_f32(((const uint16_t *)src)[idx]);
  float f = ((const float *)src)[idx];
  if (src_kind == FSO_SRC_F32_AS_BF16) return fso_bf16_to_f32(fso_f32_to_bf16(f));
  return f;
}

/* The clamp floor 1e-12 as the reference applies it.  `clamp(min=1e-12)` on a
 * bf16 tensor rounds the floor to bf16 (tests/test_flex_shard_fp8_allgather.py
 * :42,71-76); on an fp32 tensor it is the fp32 rounding of 1e-12.  The fp32
 * mode is what a quantizer that upcasts first would use. */
static inline double fso_eps(int src_kind, int eps_mode) {
  if (eps_mode == FSO_EPS_FP32 || src_kind == FSO_SRC_F32) return (double)1e-12f;
  return (double)fso_bf16_to_f32(fso_f32_to_bf16(1e-12f));
}

/*
 * Blockwise FP8 quantization of a row-major [rows, in_dim] matrix.
 * Follows tests/test_flex_shard_fp8_allgather.py:45-90 (the eager function the
 * reference's own test equates with its production kernel, :1231-1264):
 *   amax  = max |x| over the block x block tile (zero padding never raises it)
 *   amax  = max(amax, eps)                 in the input dtype
 *   scale = float32(448.0 / float64(amax))
 *   q     = e4m3fn(clamp(float32(x) * scale, -448, 448))
 *   recip = 1.0f / scale                   float32 division
 * qdata is [rows, in_dim] bytes (row stride in_dim); scales is
 * [ceil(rows/block), ceil(in_dim/block)] float32.
 */
FSO_EXPORT int fso_quantize_blockwise(const void *src, int src_kind, int64_t rows,
                                      int64_t in_dim, int64_t src_row_stride,
                                      int64_t block, int eps_mode, uint8_t *qdata,
                                      float *scales) {
  if (rows <= 0 || in_dim <= 0 || block <= 0) return -1;
  const double eps = fso_eps(src_kind, eps_mode);
  const int64_t tiles_c = (in_dim + block - 1) / block;
  const int64_t tiles_r = (rows + block - 1) / block;
  for (int64_t tr = 0; tr < tiles_r; ++tr) {
    const int64_t r0 = tr * block, r1 = r0 + block < rows ? r0 + block : rows;
    for (int64_t tc = 0; tc < tiles_c; ++tc) {
      const int64_t c0 = tc * block, c1 = c0 + block < in_dim ? c0 + block : in_dim;
      float amax = 0.0f;
      int saw_nan = 0;
      for (int64_t r = r0; r < r1; ++r)
        for (int64_t c = c0; c < c1; ++c) {
          float v = fabsf(fso_load(src, src_kind, r * src_row_stride + c));
          if (isnan(v)) saw_nan = 1;
          if (v > amax) amax = v;
        }
      double amax_d = saw_nan ? (double)NAN : (double)amax;
      if (amax_d < eps) amax_d = eps; /* NaN compares false and stays NaN */
      const float scale = (float)(448.0 / amax_d);
      for (int64_t r = r0; r < r1; ++r)
        for (int64_t c = c0; c < c1; ++c) {
          float p = fso_load(src, src_kind, r * src_row_stride + c) * scale;
          if (p > 448.0f) p = 448.0f; /* NaN falls through both tests */
          if (p < -448.0f) p = -448.0f;
          qdata[r * in_dim + c] = fso_f32_to_e4m3fn(p);
        }
      scales[tr * tiles_c + tc] = 1.0f / scale;
    }
  }
  return 0;
}

/*
 * Blockwise dequantization to bfloat16.
 * Follows blockwise_fp8/blockwise_fp8_weight.py:25-54 and :121-127:
 * float32(q) * recip_scale(tile) in fp32, then one rounding to the weight
 * dtype.  out_kind 0 writes bf16 (uint16 bits), 1 writes float32.
 */
FSO_EXPORT int fso_dequant_blockwise(const uint8_t *qdata, const float *scales,
                                     int64_t rows, int64_t in_dim, int64_t block,
                                     int out_kind, void *out) {
  if (rows <= 0 || in_dim <= 0 || block <= 0) return -1;
  const int64_t tiles_c = (in_dim + block - 1) / block;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < in_dim; ++c) {
      float v = fso_e4m3fn_to_f32(qdata[r * in_dim + c]) *
                scales[(r / block) * tiles_c + c / block];
      if (out_kind == 0)
        ((uint16_t *)out)[r * in_dim + c] = fso_f32_to_bf16(v);
      else
        ((float *)out)[r * in_dim + c] = v;
    }
  return 0;
}

/* ------------------------------------------------------------ byte segments */

/* out[dst_off[s] + i] = src[src_off[s] + i], i < nbytes[s]
 * (custom_placements/_copy_kernels.py:123-142). */
FSO_EXPORT void fso_copy_segments(const uint8_t *src, uint8_t *out, const int64_t *src_off,
                                  const int64_t *nbytes, const int64_t *dst_off,
                                  int64_t nsegments) {
  for (int64_t s = 0; s < nsegments; ++s)
    memmove(out + dst_off[s], src + src_off[s], (size_t)nbytes[s]);
}

/* Zero-fill destination segments (custom_placements/_copy_kernels.py:145-161). */
FSO_EXPORT void fso_zero_segments(uint8_t *out, const int64_t *nbytes, const int64_t *dst_off,
                                  int64_t nsegments) {
  for (int64_t s = 0; s < nsegments; ++s) memset(out + dst_off[s], 0, (size_t)nbytes[s]);
}

/* ---------------------------------------------------------------- gradients */

/* acc[i] = acc[i] + float32(g[i]) with g in bf16: one microbatch of the fp32
 * gradient accumulation (flex_shard/bucket_runtime.py:931-933; policy
 * flex_shard/bucket_storage.py:59-77). */
FSO_EXPORT void fso_accumulate_bf16(float *acc, const uint16_t *g, int64_t n) {
  for (int64_t i = 0; i < n; ++i) acc[i] = acc[i] + fso_bf16_to_f32(g[i]);
}

/* Single-GPU stand-in for the reduce-scatter of custom_placements/utils.py
 * :157-172 on rank `rank`: a left fold over contributions r = 0..W-1 of the
 * elements [col0, col0+n) of each contribution's row `rank`.
 *   mode 0: SUM             out = ((x0 + x1) + x2) + ...
 *   mode 1: pre-multiply    out = ((x0*f + x1*f) + ...)      (premul-sum, :134)
 *   mode 2: post-multiply   out = (((x0 + x1) + ...)) * f
 *   mode 3: post-divide     out = (((x0 + x1) + ...)) / f    (output.div_, :172)
 * rows[r] points at contribution r's element 0 of the wanted range. */
FSO_EXPORT void fso_reduce_rows_f32(float *out, const float *const *rows, int64_t world,
                                    int64_t n, int mode, float factor) {
  for (int64_t i = 0; i < n; ++i) {
    float s = mode == 1 ? rows[0][i] * factor : rows[0][i];
    for (int64_t r = 1; r < world; ++r) s = s + (mode == 1 ? rows[r][i] * factor : rows[r][i]);
    if (mode == 2) s = s * factor;
    if (mode == 3) s = s / factor;
    out[i] = s;
  }
}

/* ------------------------------------------------------------ Newton-Schulz */

/* C = round_bf16(alpha * (A @ B^T or A @ B) + beta * D), fp32 accumulation in
 * k order; operands are bf16 bit patterns, row-major.  Small sizes only. */
static void fso_gemm_bf16(const uint16_t *A, const uint16_t *B, int transB, const uint16_t *D,
                          float alpha, float beta, int64_t M, int64_t N, int64_t K,
                          uint16_t *C) {
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float b = transB ? fso_bf16_to_f32(B[j * K + k]) : fso_bf16_to_f32(B[k * N + j]);
        acc += fso_bf16_to_f32(A[i * K + k]) * b;
      }
      float v = alpha * acc;
      if (D) v += beta * fso_bf16_to_f32(D[i * N + j]);
      C[i * N + j] = fso_f32_to_bf16(v);
    }
}

/*
 * Quintic Newton-Schulz on one [rows, cols] matrix with rows <= cols, in
 * bfloat16 with fp32 accumulation (dist_muon/optimizer.py:2120-2151, 2-D
 * branch): X /= max(||X||_F, eps); repeat: A = X X^T; B = b A + c A A;
 * X = a X + B X, every product rounded to bf16.  The caller transposes tall
 * inputs, as the reference does.  x holds bf16 bits and is updated in place.
 * The norm is accumulated in double and rounded to bf16, the division is done
 * per element in fp32 and rounded to bf16 (torch's bf16 div_ computes in fp32).
 */
FSO_EXPORT int fso_newton_schulz_bf16(uint16_t *x, int64_t rows, int64_t cols, float a,
                                      float b, float c, int steps, float eps) {
  if (rows <= 0 || cols <= 0 || rows > cols) return -1;
  double ss = 0.0;
  for (int64_t i = 0; i < rows * cols; ++i) {
    double v = fso_bf16_to_f32(x[i]);
    ss += v * v;
  }
  float norm = fso_bf16_to_f32(fso_f32_to_bf16((float)sqrt(ss)));
  if (norm < eps) norm = fso_bf16_to_f32(fso_f32_to_bf16(eps));
  for (int64_t i = 0; i < rows * cols; ++i)
    x[i] = fso_f32_to_bf16(fso_bf16_to_f32(x[i]) / norm);
  uint16_t *gram = (uint16_t *)malloc(sizeof(uint16_t) * rows * rows);
  uint16_t *upd = (uint16_t *)malloc(sizeof(uint16_t) * rows * rows);
  uint16_t *nx = (uint16_t *)malloc(sizeof(uint16_t) * rows * cols);
  if (!gram || !upd || !nx) {
    free(gram);
    free(upd);
    free(nx);
    return -2;
  }
  for (int s = 0; s < steps; ++s) {
    fso_gemm_bf16(x, x, 1, NULL, 1.0f, 0.0f, rows, rows, cols, gram);
    fso_gemm_bf16(gram, gram, 0, gram, c, b, rows, rows, rows, upd);
    fso_gemm_bf16(upd, x, 0, x, 1.0f, a, rows, cols, rows, nx);
    memcpy(x, nx, sizeof(uint16_t) * rows * cols);
  }
  free(gram);
  free(upd);
  free(nx);
  return 0;
}
