// Unpack of gathered rank rows: byte compaction into the parameter-ordered
// buffer fused with blockwise dequantization to bf16 (or fp32), one pass over
// the FP8 bytes.
//
// A workgroup owns one block x block tile of one (rank, parameter) chunk.  For
// block = 128 and 16-byte friendly addresses each thread moves 8 FP8 bytes
// per row pass: one 8-byte load, one 8-byte store into the compact buffer,
// four v_cvt_pk_f32_fp8 + multiplies by the tile's reciprocal scale, and one
// 16-byte bf16 store.  Any other block size or alignment (rank rows at odd
// byte offsets inside a mixed bucket) takes an element-wise path.
#include "common.hpp"

namespace fsh {
namespace {

constexpr int kThreads = 256;

typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float load_f32_any(const uint8_t* p) {
  if ((reinterpret_cast<uintptr_t>(p) & 3) == 0) return *reinterpret_cast<const float*>(p);
  uint32_t u = static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8) |
               (static_cast<uint32_t>(p[2]) << 16) | (static_cast<uint32_t>(p[3]) << 24);
  return u32_as_f32(u);
}

__device__ __forceinline__ void store_f32_any(uint8_t* p, float f) {
  if ((reinterpret_cast<uintptr_t>(p) & 3) == 0) {
    *reinterpret_cast<float*>(p) = f;
    return;
  }
  const uint32_t u = f32_as_u32(f);
  p[0] = static_cast<uint8_t>(u);
  p[1] = static_cast<uint8_t>(u >> 8);
  p[2] = static_cast<uint8_t>(u >> 16);
  p[3] = static_cast<uint8_t>(u >> 24);
}

// Four FP8 bytes of `w` -> four floats times `s`.
__device__ __forceinline__ void dequant4(uint32_t w, float s, float* out) {
  const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w), false);
  const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(w), true);
  out[0] = lo.x * s;
  out[1] = lo.y * s;
  out[2] = hi.x * s;
  out[3] = hi.y * s;
}

template <int DQ>  // FSH_DT_BF16, FSH_DT_F32 or FSH_DT_F16
__global__ __launch_bounds__(kThreads) void unpack_dequant_kernel(
    const uint8_t* __restrict__ rows, const fsh_unpack_chunk* __restrict__ chunks,
    const int64_t* __restrict__ tile_starts, int nchunks, uint8_t* __restrict__ compact,
    uint8_t* __restrict__ dequant, int block) {
  const int64_t bid = blockIdx.x;
  // Largest c with tile_starts[c] <= bid.  Up to 64 chunks are resolved in one
  // memory round trip (a lane per chunk and a ballot) instead of a dependent
  // chain of binary-search probes; tile_starts is ascending, so the count of
  // entries <= bid is the index plus one.
  int lo = 0;
  if (nchunks <= 64) {
    const int l = threadIdx.x & 63;
    const bool below = l < nchunks && tile_starts[l] <= bid;
    lo = __builtin_popcountll(__ballot(below)) - 1;
  } else {
    int hi = nchunks - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (tile_starts[mid] <= bid)
        lo = mid;
      else
        hi = mid - 1;
    }
  }
  const fsh_unpack_chunk ch = chunks[lo];
  const int64_t tiles_c = (ch.in_dim + block - 1) / block;
  const int64_t t = bid - tile_starts[lo];
  const int64_t tr = t / tiles_c, tc = t - tr * tiles_c;
  const int tid = threadIdx.x;
  constexpr int kElem = DQ == FSH_DT_F32 ? 4 : 2;

  const float scale = load_f32_any(rows + ch.src_scale_offset + 4 * (tr * tiles_c + tc));
  if (compact != nullptr && tid == 0)
    store_f32_any(compact + ch.dst_scale_offset + 4 * (tr * tiles_c + tc), scale);

  const uint8_t* src = rows + ch.src_qdata_offset;
  uint8_t* cq = compact ? compact + ch.dst_qdata_offset : nullptr;
  uint8_t* dq = dequant ? dequant + ch.dst_dequant_offset * kElem : nullptr;
  const uintptr_t addr_bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(cq) |
                              reinterpret_cast<uintptr_t>(dq);
  const bool fast = block == 128 && (ch.in_dim & 15) == 0 && (addr_bits & 15) == 0;

  if (fast) {
    // 16 threads per tile row, 8 FP8 bytes each: every load and store
    // instruction of a wave then covers whole contiguous row segments (128 B
    // of FP8, 256 B of bf16), which the memory pipeline needs for full-width
    // requests.  16 rows per pass, 8 passes, all loads issued up front; rows
    // past the chunk's end are clamped for the load and skipped for the stores.
    const int g = tid & 15, r0 = tid >> 4;
    const int64_t col = tc * 128 + g * 8;
    if (col >= ch.in_dim) return;
    u32x2 vin[8];
    int64_t idxs[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t row = tr * 128 + r0 + 16 * k;
      idxs[k] = (row < ch.rows ? row : ch.rows - 1) * ch.in_dim + col;
      // A plain load: with the nontemporal hint this kernel, three quarters of
      // whose traffic are stores, measured 13 % slower on rows from HBM and
      // 25 % slower on rows still in the last-level cache (where a gather
      // has just written them).
      vin[k] = *reinterpret_cast<const u32x2*>(src + idxs[k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (tr * 128 + r0 + 16 * k >= ch.rows) break;
      const int64_t idx = idxs[k];
      const u32x2 v = vin[k];
      if (cq) store_stream_u32x2(cq + idx, v.x, v.y);
      if (dq) {
        float f[8];
        dequant4(v.x, scale, f);
        dequant4(v.y, scale, f + 4);
        if (DQ == FSH_DT_BF16) {
          u32x4 o;
          o.x = f32_to_bf16_bits(f[0]) | (f32_to_bf16_bits(f[1]) << 16);
          o.y = f32_to_bf16_bits(f[2]) | (f32_to_bf16_bits(f[3]) << 16);
          o.z = f32_to_bf16_bits(f[4]) | (f32_to_bf16_bits(f[5]) << 16);
          o.w = f32_to_bf16_bits(f[6]) | (f32_to_bf16_bits(f[7]) << 16);
          store_stream_u32x4(dq + idx * 2, o);
        } else if (DQ == FSH_DT_F16) {
          u32x4 o;
          o.x = f32_to_f16_bits(f[0]) | (f32_to_f16_bits(f[1]) << 16);
          o.y = f32_to_f16_bits(f[2]) | (f32_to_f16_bits(f[3]) << 16);
          o.z = f32_to_f16_bits(f[4]) | (f32_to_f16_bits(f[5]) << 16);
          o.w = f32_to_f16_bits(f[6]) | (f32_to_f16_bits(f[7]) << 16);
          store_stream_u32x4(dq + idx * 2, o);
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            u32x4 o = {f32_as_u32(f[4 * j]), f32_as_u32(f[4 * j + 1]), f32_as_u32(f[4 * j + 2]),
                       f32_as_u32(f[4 * j + 3])};
            store_stream_u32x4(dq + idx * 4 + 16 * j, o);
          }
        }
      }
    }
    return;
  }

  // Element-wise path.
  const int64_t row0 = tr * block, col0 = tc * block;
  const int64_t nrows = (ch.rows - row0) < block ? (ch.rows - row0) : block;
  const int64_t ncols = (ch.in_dim - col0) < block ? (ch.in_dim - col0) : block;
  for (int64_t i = tid; i < nrows * ncols; i += kThreads) {
    const int64_t idx = (row0 + i / ncols) * ch.in_dim + col0 + i % ncols;
    const uint8_t b = src[idx];
    if (cq) cq[idx] = b;
    if (dq) {
      const float f = __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(b), 0) * scale;
      if (DQ == FSH_DT_BF16)
        reinterpret_cast<uint16_t*>(dq)[idx] = static_cast<uint16_t>(f32_to_bf16_bits(f));
      else if (DQ == FSH_DT_F16)
        reinterpret_cast<uint16_t*>(dq)[idx] = static_cast<uint16_t>(f32_to_f16_bits(f));
      else
        reinterpret_cast<float*>(dq)[idx] = f;
    }
  }
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_unpack_dequant(const void* rows_dev, const fsh_unpack_chunk* chunks_dev,
                               const int64_t* tile_starts_dev, int32_t nchunks, int64_t total_tiles,
                               void* compact_dev, void* dequant_dev, int32_t dequant_dtype,
                               int32_t block, void* stream) {
  using namespace fsh;
  if (nchunks < 0 || total_tiles < 0) return fail(FSH_EINVAL, "fsh_unpack_dequant: negative size");
  if (block <= 0) return fail(FSH_EINVAL, "fsh_unpack_dequant: block must be positive, got %d", block);
  if (nchunks == 0 || total_tiles == 0) return FSH_OK;
  if (!rows_dev || !chunks_dev || !tile_starts_dev) return fail(FSH_EINVAL, "fsh_unpack_dequant: null pointer");
  if (!compact_dev && !dequant_dev) return fail(FSH_EINVAL, "fsh_unpack_dequant: nothing to write");
  if (dequant_dtype != FSH_DT_BF16 && dequant_dtype != FSH_DT_F32 && dequant_dtype != FSH_DT_F16)
    return fail(FSH_EINVAL, "fsh_unpack_dequant: unsupported dequant dtype %d", dequant_dtype);
  if (dequant_dev && !aligned(dequant_dev, dequant_dtype == FSH_DT_F32 ? 4 : 2))
    return fail(FSH_EINVAL, "fsh_unpack_dequant: dequant buffer misaligned for its dtype");
  if (total_tiles > 0x7FFFFFFFLL)
    return fail(FSH_ENOTSUP, "fsh_unpack_dequant: %lld tiles exceed the grid limit", (long long)total_tiles);
  const dim3 g(static_cast<uint32_t>(total_tiles)), b(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dequant_dtype == FSH_DT_BF16)
    hipLaunchKernelGGL((unpack_dequant_kernel<FSH_DT_BF16>), g, b, 0, s, static_cast<const uint8_t*>(rows_dev),
                       chunks_dev, tile_starts_dev, nchunks, static_cast<uint8_t*>(compact_dev),
                       static_cast<uint8_t*>(dequant_dev), block);
  else if (dequant_dtype == FSH_DT_F16)
    hipLaunchKernelGGL((unpack_dequant_kernel<FSH_DT_F16>), g, b, 0, s, static_cast<const uint8_t*>(rows_dev),
                       chunks_dev, tile_starts_dev, nchunks, static_cast<uint8_t*>(compact_dev),
                       static_cast<uint8_t*>(dequant_dev), block);
  else
    hipLaunchKernelGGL((unpack_dequant_kernel<FSH_DT_F32>), g, b, 0, s, static_cast<const uint8_t*>(rows_dev),
                       chunks_dev, tile_starts_dev, nchunks, static_cast<uint8_t*>(compact_dev),
                       static_cast<uint8_t*>(dequant_dev), block);
  return check_launch("fsh_unpack_dequant");
}
