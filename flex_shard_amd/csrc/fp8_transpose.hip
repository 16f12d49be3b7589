// Operand preparation for the backward products of the blockwise FP8 linear:
// both need an operand whose contraction index is contiguous in memory.
//
//   fp8_transpose_kernel       dst[c][r] = src[r][c] for a byte matrix (the
//                              gathered weight, read along its output index
//                              by the input-gradient product)
//   act_quant_128x1_t_kernel   quantizes every run of 128 consecutive ROWS of
//                              a column of a bf16 matrix and writes the bytes
//                              transposed, q[c][r]; serves both operands of
//                              the weight-gradient product (contraction over
//                              tokens)
//
// Both work on 128 x 128 tiles through LDS: rows go in as they are read
// (16-byte global loads along the source rows), and come out along the
// source columns as 16-byte runs of 16 source rows each.
#include "common.hpp"

namespace fsh {
namespace {

constexpr int kTileDim = 128;
constexpr int kTransposeThreads = 256;
// LDS pitch of a tile row in bytes: 33 dwords, so that the sixteen rows a
// lane gathers from and the eight row groups of a wave spread over the banks.
constexpr int kTilePitch = 132;

// Writes the transposed tile held in LDS (`tile[r * kTilePitch + c]`, r = tile
// row = destination column) to dst rows [c0, c0 + 128) x columns [r0, r0 + 128).
// Destination columns up to ld_dst are written (the caller zero-fills the tile
// rows past the source), destination rows past dst_rows are skipped.
__device__ __forceinline__ void store_tile_transposed(const uint8_t* tile, uint8_t* dst, int64_t c0, int64_t r0,
                                                      int64_t dst_rows, int64_t ld_dst, int tid) {
  const int rchunk = tid & 7;  // destination bytes [16 rchunk, +16) of the row
#pragma unroll
  for (int pass = 0; pass < kTileDim / 32; ++pass) {
    const int c = pass * 32 + (tid >> 3);
    uint32_t w[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t v = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b)
        v |= static_cast<uint32_t>(tile[(16 * rchunk + 4 * d + b) * kTilePitch + c]) << (8 * b);
      w[d] = v;
    }
    const int64_t row = c0 + c, col = r0 + 16 * rchunk;
    if (row < dst_rows && col < ld_dst)  // ld_dst is a multiple of 16
      *reinterpret_cast<u32x4*>(dst + row * ld_dst + col) = u32x4{w[0], w[1], w[2], w[3]};
  }
}

struct TransposeParams {
  const uint8_t* src;
  uint8_t* dst;
  int64_t rows, cols, ld_src, ld_dst;
  int32_t tiles_c;
};

__global__ __launch_bounds__(kTransposeThreads) void fp8_transpose_kernel(const TransposeParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileDim * kTilePitch];
  const int tid = threadIdx.x;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x / p.tiles_c) * kTileDim;
  const int64_t c0 = static_cast<int64_t>(blockIdx.x % p.tiles_c) * kTileDim;
  const int chunk = tid & 7;
  u32x4 v[4];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int64_t row = r0 + pass * 32 + (tid >> 3), col = c0 + chunk * 16;
    v[pass] = u32x4{0, 0, 0, 0};
    if (row < p.rows && col < p.cols) {  // cols is a multiple of 16
      v[pass] = load_stream_u32x4(p.src + row * p.ld_src + col);
    }
  }
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(tile + (pass * 32 + (tid >> 3)) * kTilePitch + chunk * 16);
    dst[0] = v[pass].x; dst[1] = v[pass].y; dst[2] = v[pass].z; dst[3] = v[pass].w;
  }
  __syncthreads();
  store_tile_transposed(tile, p.dst, c0, r0, p.cols, p.ld_dst, tid);
}

struct ActQuantTParams {
  const uint8_t* x;
  uint8_t* q;      // [cols][ldq]
  float* scales;   // [ldq / 128][cols]
  int64_t rows, cols, ldx, ldq;
  int32_t tiles_c;
  float eps;
  // the row-run outputs of the dual kernel: q_row [rows][ldq_row], scales_row [ldq_row / 128][rows]
  uint8_t* q_row;
  float* scales_row;
  int64_t ldq_row;
};

// Thread t loads columns [8 (t & 15), +8) of tile rows (t >> 4) + 16 k, k = 0..7.
// kAlsoRowRuns: the same tile also leaves quantized in runs of 128 along its
// rows (the arithmetic and the outputs of act_quant_1x128_kernel), so an
// operand needed in both forms is read once.  A tile row's 128 columns lie in
// one row of 16 lanes, whose maximum takes four DPP steps.
template <bool kAlsoRowRuns>
__global__ __launch_bounds__(kTransposeThreads) void act_quant_128x1_t_kernel(const ActQuantTParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileDim * kTilePitch];
  __shared__ __attribute__((aligned(16))) uint16_t col_max[16 * kTileDim];
  __shared__ __attribute__((aligned(16))) float col_scale[kTileDim];
  __shared__ float row_recip[kAlsoRowRuns ? kTileDim : 1];
  const int tid = threadIdx.x;
  const int cg = tid & 15, rl = tid >> 4;
  const int64_t rb = blockIdx.x / p.tiles_c;
  const int64_t r0 = rb * kTileDim, c0 = static_cast<int64_t>(blockIdx.x % p.tiles_c) * kTileDim;
  const int64_t col = c0 + cg * 8;

  u32x4 v[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t row = r0 + rl + 16 * k;
    v[k] = u32x4{0, 0, 0, 0};
    if (row < p.rows && col < p.cols) v[k] = load_stream_u32x4(p.x + (row * p.ldx + col) * 2);  // cols % 8 == 0
  }
  if (kAlsoRowRuns) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t row = r0 + rl + 16 * k;
      uint32_t mr = pk_max_u16(v[k].x & 0x7FFF7FFFu, v[k].y & 0x7FFF7FFFu);
      mr = pk_max_u16(mr, v[k].z & 0x7FFF7FFFu);
      mr = pk_max_u16(mr, v[k].w & 0x7FFF7FFFu);
      const uint32_t lo = mr & 0xFFFFu, hi = mr >> 16;
      mr = row16_max_u32(lo > hi ? lo : hi);
      float scale, recip;
      tile_scale(bf16_bits_to_f32(mr), p.eps, scale, recip);
      if (cg == 0) row_recip[rl + 16 * k] = recip;
      if (row < p.rows && col < p.ldq_row) {  // columns past `cols` hold zeros: the pad of the last run
        const uint32_t d[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float e0 = u32_as_f32(d[j] << 16) * scale;
          const float e1 = u32_as_f32(d[j] & 0xFFFF0000u) * scale;
          w[j >> 1] = cvt2_fp8(e0, e1, w[j >> 1], (j & 1) != 0);
        }
        store_stream_u32x2(p.q_row + row * p.ldq_row + col, w[0], w[1]);
      }
    }
  }
  // Largest magnitude (bf16 bit pattern) of the thread's eight rows, per column.
  uint32_t m[4] = {0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    m[0] = pk_max_u16(m[0], v[k].x & 0x7FFF7FFFu);
    m[1] = pk_max_u16(m[1], v[k].y & 0x7FFF7FFFu);
    m[2] = pk_max_u16(m[2], v[k].z & 0x7FFF7FFFu);
    m[3] = pk_max_u16(m[3], v[k].w & 0x7FFF7FFFu);
  }
  *reinterpret_cast<u32x4*>(col_max + rl * kTileDim + cg * 8) = u32x4{m[0], m[1], m[2], m[3]};
  __syncthreads();
  if (tid < kTileDim) {
    uint32_t best = 0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const uint32_t candidate = col_max[r * kTileDim + tid];
      best = candidate > best ? candidate : best;
    }
    float scale, recip;
    tile_scale(bf16_bits_to_f32(best), p.eps, scale, recip);
    col_scale[tid] = scale;
    if (c0 + tid < p.cols) p.scales[rb * p.cols + c0 + tid] = recip;
    // (row_recip was filled before the first barrier above)
    if (kAlsoRowRuns && r0 + tid < p.rows) p.scales_row[(c0 / kTileDim) * p.rows + r0 + tid] = row_recip[tid];
  }
  __syncthreads();
  const f32x4 s_lo = *reinterpret_cast<const f32x4*>(col_scale + cg * 8);
  const f32x4 s_hi = *reinterpret_cast<const f32x4*>(col_scale + cg * 8 + 4);
  const float s[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const uint32_t d[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float e0 = u32_as_f32(d[j] << 16) * s[2 * j];
      const float e1 = u32_as_f32(d[j] & 0xFFFF0000u) * s[2 * j + 1];
      w[j >> 1] = cvt2_fp8(e0, e1, w[j >> 1], (j & 1) != 0);
    }
    uint32_t* dst = reinterpret_cast<uint32_t*>(tile + (rl + 16 * k) * kTilePitch + cg * 8);
    dst[0] = w[0];
    dst[1] = w[1];
  }
  __syncthreads();
  store_tile_transposed(tile, p.q, c0, r0, p.cols, p.ldq, tid);
}

float floor_for(int32_t eps_mode) {
  const float eps32 = 1e-12f;
  uint32_t bits;
  memcpy(&bits, &eps32, 4);
  bits = (bits + 0x7FFFu + ((bits >> 16) & 1u)) & 0xFFFF0000u;
  float eps_bf16;
  memcpy(&eps_bf16, &bits, 4);
  return eps_mode == FSH_EPS_FP32 ? eps32 : eps_bf16;
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_fp8_transpose(const void* src_dev, int64_t rows, int64_t cols, int64_t ld_src, void* dst_dev,
                              int64_t ld_dst, void* stream) {
  using namespace fsh;
  if (rows < 0 || cols < 0) return fail(FSH_EINVAL, "fsh_fp8_transpose: negative shape");
  if (rows == 0 || cols == 0) return FSH_OK;
  if (!src_dev || !dst_dev) return fail(FSH_EINVAL, "fsh_fp8_transpose: null pointer");
  if (ld_src < cols || ld_dst < rows)
    return fail(FSH_EINVAL, "fsh_fp8_transpose: ld_src %lld < cols %lld or ld_dst %lld < rows %lld", (long long)ld_src,
                (long long)cols, (long long)ld_dst, (long long)rows);
  if (cols % 16 || ld_src % 16 || ld_dst % 16 || !aligned(src_dev, 16) || !aligned(dst_dev, 16))
    return fail(FSH_ENOTSUP, "fsh_fp8_transpose: cols and both leading dimensions must be multiples of 16, pointers 16-byte aligned");
  if (ld_dst > ceil_div(rows, (int64_t)kTileDim) * kTileDim)
    return fail(FSH_ENOTSUP, "fsh_fp8_transpose: ld_dst %lld exceeds rows %lld rounded up to 128 (only that much is zero-filled)",
                (long long)ld_dst, (long long)rows);
  TransposeParams p;
  p.src = static_cast<const uint8_t*>(src_dev);
  p.dst = static_cast<uint8_t*>(dst_dev);
  p.rows = rows; p.cols = cols; p.ld_src = ld_src; p.ld_dst = ld_dst;
  const int64_t tiles_c = ceil_div(cols, (int64_t)kTileDim);
  const int64_t grid = ceil_div(rows, (int64_t)kTileDim) * tiles_c;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_fp8_transpose: too many tiles");
  p.tiles_c = static_cast<int32_t>(tiles_c);
  hipLaunchKernelGGL(fp8_transpose_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kTransposeThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch("fp8_transpose_kernel");
}

FSH_API int fsh_act_quant_128x1_transposed(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_dev,
                                           int64_t ldq, float* scales_dev, int32_t eps_mode, void* stream) {
  using namespace fsh;
  if (rows < 0 || cols < 0) return fail(FSH_EINVAL, "fsh_act_quant_128x1_transposed: negative shape");
  if (rows == 0 || cols == 0) return FSH_OK;
  if (!x_dev || !q_dev || !scales_dev) return fail(FSH_EINVAL, "fsh_act_quant_128x1_transposed: null pointer");
  if (eps_mode != FSH_EPS_INPUT_DTYPE && eps_mode != FSH_EPS_FP32)
    return fail(FSH_EINVAL, "fsh_act_quant_128x1_transposed: unknown eps_mode %d", eps_mode);
  const int64_t padded = ceil_div(rows, (int64_t)kTileDim) * kTileDim;
  if (ldx < cols || ldq != padded)
    return fail(FSH_EINVAL,
                "fsh_act_quant_128x1_transposed: ldx %lld < cols %lld, or ldq %lld is not rows rounded up to 128 (%lld)",
                (long long)ldx, (long long)cols, (long long)ldq, (long long)padded);
  if (cols % 8 || ldx % 8 || !aligned(x_dev, 16) || !aligned(q_dev, 16) || !aligned(scales_dev, 4))
    return fail(FSH_ENOTSUP, "fsh_act_quant_128x1_transposed: cols and ldx must be multiples of 8, x and q 16-byte aligned");
  ActQuantTParams p;
  p.x = static_cast<const uint8_t*>(x_dev);
  p.q = static_cast<uint8_t*>(q_dev);
  p.scales = scales_dev;
  p.rows = rows; p.cols = cols; p.ldx = ldx; p.ldq = ldq;
  p.eps = floor_for(eps_mode);
  p.q_row = nullptr; p.scales_row = nullptr; p.ldq_row = 0;
  const int64_t tiles_c = ceil_div(cols, (int64_t)kTileDim);
  const int64_t grid = (padded / kTileDim) * tiles_c;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_act_quant_128x1_transposed: too many tiles");
  p.tiles_c = static_cast<int32_t>(tiles_c);
  hipLaunchKernelGGL(act_quant_128x1_t_kernel<false>, dim3(static_cast<uint32_t>(grid)), dim3(kTransposeThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch("act_quant_128x1_t_kernel");
}

FSH_API int fsh_act_quant_both(const void* x_dev, int64_t rows, int64_t cols, int64_t ldx, void* q_row_dev,
                               int64_t ldq_row, float* scales_row_dev, void* q_col_dev, int64_t ldq_col,
                               float* scales_col_dev, int32_t eps_mode, void* stream) {
  using namespace fsh;
  if (rows < 0 || cols < 0) return fail(FSH_EINVAL, "fsh_act_quant_both: negative shape");
  if (rows == 0 || cols == 0) return FSH_OK;
  if (!x_dev || !q_row_dev || !scales_row_dev || !q_col_dev || !scales_col_dev)
    return fail(FSH_EINVAL, "fsh_act_quant_both: null pointer");
  if (eps_mode != FSH_EPS_INPUT_DTYPE && eps_mode != FSH_EPS_FP32)
    return fail(FSH_EINVAL, "fsh_act_quant_both: unknown eps_mode %d", eps_mode);
  const int64_t padded_rows = ceil_div(rows, (int64_t)kTileDim) * kTileDim;
  const int64_t padded_cols = ceil_div(cols, (int64_t)kTileDim) * kTileDim;
  if (ldx < cols || ldq_col != padded_rows || ldq_row != padded_cols)
    return fail(FSH_EINVAL,
                "fsh_act_quant_both: ldx %lld < cols %lld, ldq_col %lld is not rows rounded up to 128 (%lld), or "
                "ldq_row %lld is not cols rounded up to 128 (%lld)",
                (long long)ldx, (long long)cols, (long long)ldq_col, (long long)padded_rows, (long long)ldq_row,
                (long long)padded_cols);
  if (cols % 8 || ldx % 8 || !aligned(x_dev, 16) || !aligned(q_col_dev, 16) || !aligned(q_row_dev, 8) ||
      !aligned(scales_row_dev, 4) || !aligned(scales_col_dev, 4))
    return fail(FSH_ENOTSUP, "fsh_act_quant_both: cols and ldx must be multiples of 8, x and q_col 16-byte and q_row 8-byte aligned");
  ActQuantTParams p;
  p.x = static_cast<const uint8_t*>(x_dev);
  p.q = static_cast<uint8_t*>(q_col_dev);
  p.scales = scales_col_dev;
  p.rows = rows; p.cols = cols; p.ldx = ldx; p.ldq = ldq_col;
  p.eps = floor_for(eps_mode);
  p.q_row = static_cast<uint8_t*>(q_row_dev);
  p.scales_row = scales_row_dev;
  p.ldq_row = ldq_row;
  const int64_t tiles_c = padded_cols / kTileDim;
  const int64_t grid = (padded_rows / kTileDim) * tiles_c;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_act_quant_both: too many tiles");
  p.tiles_c = static_cast<int32_t>(tiles_c);
  hipLaunchKernelGGL(act_quant_128x1_t_kernel<true>, dim3(static_cast<uint32_t>(grid)), dim3(kTransposeThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch("act_quant_128x1_t_kernel<true>");
}
