// Newton-Schulz orthogonalization for Muon on gfx950 matrix cores.
//
// Everything is built from one batched "NT" GEMM, C = bf16(alpha*A*B^T +
// beta*D) with both operands k-contiguous, so every MFMA operand is one
// 16-byte LDS read.  To keep all three products of an iteration in that
// form the iterate is carried in both orientations, X [s, l] and X^T [l, s]
// (s <= l):
//   G  = X X^T                 A = X,  B = X
//   P  = b G + c G G           A = G,  B = G   (G symmetric, so G^T = G)
//   X' = a X + P X             A = P,  B = X^T; the epilogue writes X' in
//                              place and X'^T into the other X^T buffer.
// A tall input is its own X^T, so no transpose kernel is needed in either
// case, and the result lands in the caller's buffer without a copy.
//
// GEMM kernel: 256 threads (2x2 wavefronts), 128x128 block tile, BK = 32,
// v_mfma_f32_32x32x16_bf16, each wave a 64x64 tile (2x2 MFMA tiles, 64 fp32
// accumulators per lane).  Global->register->LDS double buffering with one
// barrier per k-tile; LDS rows padded by 16 bytes so the 64 lanes of a
// ds_read_b128 hit distinct banks.
#include "common.hpp"

namespace fsh {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct GemmParams {
  const uint16_t* A;
  const uint16_t* B;
  const uint16_t* D;
  uint16_t* C;
  uint16_t* Ct;
  int64_t M, N, K;
  int64_t lda, ldb, ldd, ldc, ldct;
  int64_t sA, sB, sD, sC, sCt;
  float alpha, beta;
  int32_t tiles_m, tiles_n;
};

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int kGemmThreads = 256;
constexpr int kLdsStride = BK + 8;  // bf16 elements per LDS row (80 bytes)

__global__ __launch_bounds__(kGemmThreads) void gemm_nt_kernel(const GemmParams p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[2][(BM + BN) * kLdsStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t batch = blockIdx.y;

  // Tiles are numbered so that the 8 workgroups that land on one XCD in a row
  // (round-robin dispatch) walk down one column block: they share the B
  // operand rows in that XCD's L2.
  const int tile = blockIdx.x;
  const int tm = tile % p.tiles_m;
  const int tn = tile / p.tiles_m;
  const int64_t m0 = static_cast<int64_t>(tm) * BM;
  const int64_t n0 = static_cast<int64_t>(tn) * BN;

  const uint16_t* A = p.A + batch * p.sA;
  const uint16_t* B = p.B + batch * p.sB;

  // Global -> register staging: 16-byte chunks, 4 per LDS row.
  constexpr int kChunksPerRow = BK / 8;
  constexpr int kChunks = BM * kChunksPerRow / kGemmThreads;  // 2 (BM == BN)
  u32x4 ra[kChunks], rb[kChunks];
  int lrow[kChunks], lkc[kChunks];
#pragma unroll
  for (int i = 0; i < kChunks; ++i) {
    const int c = tid + i * kGemmThreads;
    lrow[i] = c / kChunksPerRow;
    lkc[i] = c % kChunksPerRow;
  }

  auto load_global = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int64_t gk = k0 + lkc[i] * 8;
      const int64_t ar = m0 + lrow[i], br = n0 + lrow[i];
      ra[i] = u32x4{0, 0, 0, 0};
      rb[i] = u32x4{0, 0, 0, 0};
      if (ar < p.M && gk < p.K) ra[i] = *reinterpret_cast<const u32x4*>(A + ar * p.lda + gk);
      if (br < p.N && gk < p.K) rb[i] = *reinterpret_cast<const u32x4*>(B + br * p.ldb + gk);
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      *reinterpret_cast<u32x4*>(&smem[buf][lrow[i] * kLdsStride + lkc[i] * 8]) = ra[i];
      *reinterpret_cast<u32x4*>(&smem[buf][(BM + lrow[i]) * kLdsStride + lkc[i] * 8]) = rb[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;
  const int64_t ktiles = (p.K + BK - 1) / BK;

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int64_t kt = 0; kt < ktiles; ++kt) {
    const int buf = static_cast<int>(kt & 1);
    if (kt + 1 < ktiles) load_global((kt + 1) * BK);
    const uint16_t* As = &smem[buf][0];
    const uint16_t* Bs = &smem[buf][BM * kLdsStride];
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(&As[(wm * 64 + i * 32 + frag_row) * kLdsStride + ks * 16 + frag_k]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[j] = *reinterpret_cast<const bf16x8*>(&Bs[(wn * 64 + j * 32 + frag_row) * kLdsStride + ks * 16 + frag_k]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ktiles) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue.  Accumulator r of a 32x32 MFMA tile belongs to column lane%32
  // and row 8*(r/4) + 4*(lane/32) + r%4.
  const uint16_t* D = p.D ? p.D + batch * p.sD : nullptr;
  uint16_t* C = p.C + batch * p.sC;
  uint16_t* Ct = p.Ct ? p.Ct + batch * p.sCt : nullptr;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = n0 + wn * 64 + j * 32 + (lane & 31);
      if (col >= p.N) continue;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int64_t row_base = m0 + wm * 64 + i * 32 + 8 * b + 4 * (lane >> 5);
        uint32_t packed[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int64_t row = row_base + t;
          float v = p.alpha * acc[i][j][4 * b + t];
          if (D != nullptr && row < p.M) v += p.beta * bf16_bits_to_f32(D[row * p.ldd + col]);
          packed[t] = f32_to_bf16_bits(v);
          if (row < p.M) C[row * p.ldc + col] = static_cast<uint16_t>(packed[t]);
        }
        if (Ct != nullptr) {
          if (row_base + 3 < p.M) {
            *reinterpret_cast<u32x2*>(&Ct[col * p.ldct + row_base]) =
                u32x2{packed[0] | (packed[1] << 16), packed[2] | (packed[3] << 16)};
          } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
              if (row_base + t < p.M) Ct[col * p.ldct + row_base + t] = static_cast<uint16_t>(packed[t]);
          }
        }
      }
    }
}

int launch_gemm(const fsh_gemm_desc& d, hipStream_t stream) {
  if (d.m <= 0 || d.n <= 0 || d.k <= 0 || d.batch <= 0)
    return fail(FSH_EINVAL, "gemm: non-positive size (m %lld, n %lld, k %lld, batch %lld)", (long long)d.m,
                (long long)d.n, (long long)d.k, (long long)d.batch);
  if (!d.a_dev || !d.b_dev || !d.c_dev) return fail(FSH_EINVAL, "gemm: null operand");
  if (d.k % 8 || d.lda % 8 || d.ldb % 8 || d.stride_a % 8 || d.stride_b % 8 || !aligned(d.a_dev, 16) ||
      !aligned(d.b_dev, 16))
    return fail(FSH_ENOTSUP, "gemm: k, lda, ldb and batch strides must be multiples of 8 and A, B 16-byte aligned");
  if (d.lda < d.k || d.ldb < d.k || d.ldc < d.n || (d.d_dev && d.ldd < d.n) || (d.ct_dev && d.ldct < d.m))
    return fail(FSH_EINVAL, "gemm: leading dimension smaller than the row length");
  if (d.ct_dev && (d.ldct % 4 || d.stride_ct % 4 || !aligned(d.ct_dev, 8)))
    return fail(FSH_ENOTSUP, "gemm: transposed output needs ldct %% 4 == 0 and an 8-byte aligned pointer");
  if (d.batch > 65535) return fail(FSH_ENOTSUP, "gemm: batch %lld exceeds 65535", (long long)d.batch);
  GemmParams p;
  p.A = static_cast<const uint16_t*>(d.a_dev);
  p.B = static_cast<const uint16_t*>(d.b_dev);
  p.D = static_cast<const uint16_t*>(d.d_dev);
  p.C = static_cast<uint16_t*>(d.c_dev);
  p.Ct = static_cast<uint16_t*>(d.ct_dev);
  p.M = d.m; p.N = d.n; p.K = d.k;
  p.lda = d.lda; p.ldb = d.ldb; p.ldd = d.ldd; p.ldc = d.ldc; p.ldct = d.ldct;
  p.sA = d.stride_a; p.sB = d.stride_b; p.sD = d.stride_d; p.sC = d.stride_c; p.sCt = d.stride_ct;
  p.alpha = d.alpha; p.beta = d.beta;
  p.tiles_m = static_cast<int32_t>(ceil_div(d.m, BM));
  p.tiles_n = static_cast<int32_t>(ceil_div(d.n, BN));
  const int64_t tiles = static_cast<int64_t>(p.tiles_m) * p.tiles_n;
  if (tiles > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "gemm: too many tiles");
  hipLaunchKernelGGL(gemm_nt_kernel, dim3(static_cast<uint32_t>(tiles), static_cast<uint32_t>(d.batch)),
                     dim3(kGemmThreads), 0, stream, p);
  return check_launch("gemm_nt_kernel");
}

// ------------------------------------------------------- Frobenius normalize
constexpr int kNormThreads = 256;
constexpr int kNormBlocksPerMatrix = 64;

// partial[b][j] = sum of squares of a slice of matrix b (fp32, fixed order).
__global__ __launch_bounds__(kNormThreads) void sumsq_partial_kernel(const uint16_t* __restrict__ x,
                                                                    int64_t numel, float* __restrict__ partial) {
  __shared__ float lds[kNormThreads / 64];
  const int64_t b = blockIdx.y;
  const uint16_t* m = x + b * numel;
  const int64_t per = ceil_div(ceil_div(numel, (int64_t)kNormBlocksPerMatrix), 8) * 8;
  const int64_t begin = blockIdx.x * per;
  const int64_t end = (begin + per) < numel ? (begin + per) : numel;
  float s = 0.0f;
  for (int64_t i = begin + threadIdx.x; i < end; i += kNormThreads) {
    const float v = bf16_bits_to_f32(m[i]);
    s += v * v;
  }
  s = wave_sum_f32(s);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[b * kNormBlocksPerMatrix + blockIdx.x] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

// Reads matrix b of `in` ([rows, cols]), divides by max(||.||_F, eps) as bf16
// tensor ops would (norm rounded to bf16, fp32 division, bf16 result), and
// writes the result to `out_same` ([rows, cols]) and `out_t` ([cols, rows]).
// 32x32 tiles go through LDS so both writes are row-contiguous.
__global__ __launch_bounds__(kNormThreads) void normalize_dual_kernel(const uint16_t* __restrict__ in,
                                                                     uint16_t* __restrict__ out_same,
                                                                     uint16_t* __restrict__ out_t, int64_t rows,
                                                                     int64_t cols, const float* __restrict__ partial,
                                                                     float eps_bf16) {
  __shared__ uint16_t tile[32][33];
  const int64_t b = blockIdx.z;
  float total = 0.0f;
  for (int j = 0; j < kNormBlocksPerMatrix; ++j) total += partial[b * kNormBlocksPerMatrix + j];
  float norm = bf16_bits_to_f32(f32_to_bf16_bits(sqrtf(total)));
  norm = norm < eps_bf16 ? eps_bf16 : norm;
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 32, c0 = static_cast<int64_t>(blockIdx.x) * 32;
  const uint16_t* m = in + b * rows * cols;
  uint16_t* o = out_same + b * rows * cols;
  uint16_t* ot = out_t + b * rows * cols;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t r = r0 + ty + 8 * k, c = c0 + tx;
    if (r < rows && c < cols) {
      const uint16_t v = static_cast<uint16_t>(f32_to_bf16_bits(bf16_bits_to_f32(m[r * cols + c]) / norm));
      o[r * cols + c] = v;
      tile[ty + 8 * k][tx] = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t c = c0 + ty + 8 * k, r = r0 + tx;
    if (r < rows && c < cols) ot[c * rows + r] = tile[tx][ty + 8 * k];
  }
}

float bf16_round_host(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  memcpy(&f, &u, 4);
  return f;
}

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

}  // namespace
}  // namespace fsh

FSH_API int fsh_gemm_bf16_nt(const fsh_gemm_desc* desc, void* stream) {
  if (desc == nullptr) return fsh::fail(FSH_EINVAL, "fsh_gemm_bf16_nt: null descriptor");
  return fsh::launch_gemm(*desc, static_cast<hipStream_t>(stream));
}

// Workspace layout (bytes, each region 256-aligned):
//   other orientation of the iterate [batch, s*l] bf16
//   second X^T buffer                [batch, s*l] bf16
//   G                                [batch, s*s] bf16
//   P                                [batch, s*s] bf16
//   norm partials                    [batch, 64] fp32
FSH_API int64_t fsh_newton_schulz_workspace_bytes(int64_t batch, int64_t rows, int64_t cols) {
  using namespace fsh;
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  const int64_t s = rows < cols ? rows : cols, l = rows < cols ? cols : rows;
  return 2 * align256(batch * s * l * 2) + 2 * align256(batch * s * s * 2) +
         align256(batch * kNormBlocksPerMatrix * 4);
}

FSH_API int fsh_newton_schulz(void* x_dev, int64_t batch, int64_t rows, int64_t cols, float a, float b,
                              float c, int32_t steps, float eps, void* workspace_dev,
                              int64_t workspace_nbytes, void* stream_) {
  using namespace fsh;
  if (batch <= 0 || rows <= 0 || cols <= 0 || steps < 0)
    return fail(FSH_EINVAL, "fsh_newton_schulz: bad sizes (batch %lld, rows %lld, cols %lld, steps %d)",
                (long long)batch, (long long)rows, (long long)cols, steps);
  if (!x_dev || !workspace_dev) return fail(FSH_EINVAL, "fsh_newton_schulz: null pointer");
  if (rows % 8 || cols % 8)
    return fail(FSH_ENOTSUP, "fsh_newton_schulz: rows and cols must be multiples of 8, got %lld x %lld",
                (long long)rows, (long long)cols);
  if (!aligned(x_dev, 16) || !aligned(workspace_dev, 256))
    return fail(FSH_EINVAL, "fsh_newton_schulz: x must be 16-byte and workspace 256-byte aligned");
  if (batch > 65535) return fail(FSH_ENOTSUP, "fsh_newton_schulz: batch %lld exceeds 65535", (long long)batch);
  const int64_t need = fsh_newton_schulz_workspace_bytes(batch, rows, cols);
  if (workspace_nbytes < need)
    return fail(FSH_EINVAL, "fsh_newton_schulz: workspace of %lld bytes, need %lld", (long long)workspace_nbytes,
                (long long)need);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const bool tall = rows > cols;
  const int64_t s = tall ? cols : rows, l = tall ? rows : cols;
  const int64_t sl = s * l, ss = s * s;

  uint8_t* ws = static_cast<uint8_t*>(workspace_dev);
  uint16_t* w0 = reinterpret_cast<uint16_t*>(ws);
  uint16_t* w1 = reinterpret_cast<uint16_t*>(ws + align256(batch * sl * 2));
  uint16_t* G = reinterpret_cast<uint16_t*>(ws + 2 * align256(batch * sl * 2));
  uint16_t* P = reinterpret_cast<uint16_t*>(ws + 2 * align256(batch * sl * 2) + align256(batch * ss * 2));
  float* partial = reinterpret_cast<float*>(ws + 2 * align256(batch * sl * 2) + 2 * align256(batch * ss * 2));
  uint16_t* x = static_cast<uint16_t*>(x_dev);

  // X is [s, l]; XT[0], XT[1] are the two [l, s] buffers.  The caller's
  // buffer is X when the input is wide and XT[0] when it is tall.  The first
  // X^T goes to XT[steps % 2] so that the last step leaves X^T in XT[0].
  uint16_t* X = tall ? w0 : x;
  uint16_t* XT[2] = {tall ? x : w0, w1};
  int cur = steps & 1;

  hipLaunchKernelGGL(sumsq_partial_kernel, dim3(kNormBlocksPerMatrix, static_cast<uint32_t>(batch)),
                     dim3(kNormThreads), 0, stream, x, rows * cols, partial);
  if (int rc = check_launch("sumsq_partial_kernel")) return rc;
  {
    // Input is [rows, cols]; "same orientation" output is X for a wide input
    // and X^T for a tall one.
    uint16_t* same = tall ? XT[cur] : X;
    uint16_t* transposed = tall ? X : XT[cur];
    const dim3 grid(static_cast<uint32_t>(ceil_div(cols, 32)), static_cast<uint32_t>(ceil_div(rows, 32)),
                    static_cast<uint32_t>(batch));
    if (grid.y > 65535) return fail(FSH_ENOTSUP, "fsh_newton_schulz: more than %d row tiles", 65535 * 32);
    hipLaunchKernelGGL(normalize_dual_kernel, grid, dim3(kNormThreads), 0, stream, x, same, transposed, rows,
                       cols, partial, bf16_round_host(eps));
    if (int rc = check_launch("normalize_dual_kernel")) return rc;
  }

  for (int step = 0; step < steps; ++step) {
    fsh_gemm_desc g;
    memset(&g, 0, sizeof(g));
    g.batch = batch;
    // G = X X^T
    g.a_dev = X; g.b_dev = X; g.d_dev = nullptr; g.c_dev = G; g.ct_dev = nullptr;
    g.m = s; g.n = s; g.k = l; g.lda = l; g.ldb = l; g.ldc = s;
    g.stride_a = sl; g.stride_b = sl; g.stride_c = ss;
    g.alpha = 1.0f; g.beta = 0.0f;
    if (int rc = launch_gemm(g, stream)) return rc;
    // P = b G + c G G
    g.a_dev = G; g.b_dev = G; g.d_dev = G; g.c_dev = P;
    g.m = s; g.n = s; g.k = s; g.lda = s; g.ldb = s; g.ldd = s; g.ldc = s;
    g.stride_a = ss; g.stride_b = ss; g.stride_d = ss; g.stride_c = ss;
    g.alpha = c; g.beta = b;
    if (int rc = launch_gemm(g, stream)) return rc;
    // X' = a X + P X, also written transposed into the other X^T buffer
    g.a_dev = P; g.b_dev = XT[cur]; g.d_dev = X; g.c_dev = X; g.ct_dev = XT[cur ^ 1];
    g.m = s; g.n = l; g.k = s; g.lda = s; g.ldb = s; g.ldd = l; g.ldc = l; g.ldct = s;
    g.stride_a = ss; g.stride_b = sl; g.stride_d = sl; g.stride_c = sl; g.stride_ct = sl;
    g.alpha = 1.0f; g.beta = a;
    if (int rc = launch_gemm(g, stream)) return rc;
    cur ^= 1;
  }
  // cur == 0 here: for a tall input the result X^T is in the caller's buffer;
  // for a wide input X was updated in place.
  return FSH_OK;
}
