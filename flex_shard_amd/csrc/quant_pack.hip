// Fused blockwise FP8 (E4M3FN) tile quantization + packing into a rank's
// flat send payload, one launch per bucket.
//
// One workgroup (256 threads = 4 wavefronts) owns one block x block tile of
// one chunk.  For block = 128 each thread keeps its 64 tile elements in
// registers between the amax pass and the cast pass, so the tile is read from
// HBM exactly once: 16-byte loads (8 bf16), amax on raw magnitude bits with
// packed 16-bit max, a 64-lane DPP reduction plus a 4-entry LDS exchange,
// one fp64 division per tile for the scale, then v_cvt_pk_fp8_f32 and 8-byte
// stores straight into the payload.  Extra workgroups zero the payload's pad
// gaps, so nothing else has to touch the buffer.
//
// Arithmetic contract (bit-exact with the reference's eager quantizer):
//   amax   = max |x| in the quantization dtype
//   amax   = amax < eps ? eps : amax            (NaN stays NaN)
//   scale  = float(448.0 / double(amax))
//   q      = e4m3fn_rne(float(x) * scale)       (the reference's clamp to
//            +-448 never changes a finite product: |x| <= amax bounds it by
//            448 * (1 + 2^-23), which rounds to 448 either way)
//   stored = 1.0f / scale                       (IEEE fp32 division)
#include <algorithm>
#include <new>
#include <vector>

#include "common.hpp"

namespace fsh {
namespace {

constexpr int kThreads = 256;
constexpr int64_t kZeroChunk = 65536;  // bytes zeroed per pad workgroup

struct QuantChunkDev {
  const uint8_t* src;
  int64_t rows;
  int64_t in_dim;
  int64_t src_row_stride;  // elements
  int64_t qdata_offset;
  int64_t scale_offset;
  int64_t tile_begin;  // index of the chunk's first tile in the launch
  int32_t tiles_c;
  int32_t src_kind;
  int32_t fast;  // 128x128 vector path is legal for this chunk
  int32_t pad_;
};

struct QuantParams {
  QuantChunkDev chunks[FSH_MAX_QUANT_CHUNKS];
  uint8_t* payload;
  int64_t total_tiles;
  int64_t zero_begin[2];
  int64_t zero_len[2];
  float eps[5];  // indexed by src_kind
  int32_t nchunks;
  int32_t block;
};

// Workgroup-wide maximum of one magnitude word per thread.
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, uint32_t* lds) {
  v = wave_max_u32(v);
  const int tid = threadIdx.x;
  if ((tid & 63) == 0) lds[tid >> 6] = v;
  __syncthreads();
  uint32_t a = lds[0] > lds[1] ? lds[0] : lds[1];
  uint32_t b = lds[2] > lds[3] ? lds[2] : lds[3];
  return a > b ? a : b;
}

// ---------------------------------------------------------------- fast path
// Thread t owns columns 8*(t%16) .. +7 of rows (t/16) + 16k, k = 0..7.
// Per load instruction a wavefront reads four full 256-byte tile rows.

// bf16 or fp16 source, or fp32 master rounded to one of them on load: the
// tile lives in registers as 32 dwords of packed 16-bit values.  (Magnitude
// bits order like the values in both formats, NaN patterns above infinity.)
template <int KIND>
__device__ __forceinline__ void quant_tile128_bf16(const QuantChunkDev& ch, int64_t tr, int64_t tc,
                                                   uint8_t* payload, float eps, uint32_t* lds) {
  const int tid = threadIdx.x;
  const int g = tid & 15;
  const int r0 = tid >> 4;
  const int64_t row_base = tr * 128 + r0;
  const int64_t col = tc * 128 + g * 8;
  const bool col_ok = col < ch.in_dim;

  u32x4 v[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t row = row_base + 16 * k;
    v[k] = u32x4{0, 0, 0, 0};
    if (col_ok && row < ch.rows) {
      if (KIND == FSH_SRC_BF16 || KIND == FSH_SRC_F16) {
        v[k] = load_stream_u32x4(ch.src + (row * ch.src_row_stride + col) * 2);
      } else {
        const uint8_t* p = ch.src + (row * ch.src_row_stride + col) * 4;
        const f32x4 a = load_stream_f32x4(p);
        const f32x4 b = load_stream_f32x4(p + 16);
        if (KIND == FSH_SRC_F32_AS_BF16) {
          v[k].x = f32_to_bf16_bits(a.x) | (f32_to_bf16_bits(a.y) << 16);
          v[k].y = f32_to_bf16_bits(a.z) | (f32_to_bf16_bits(a.w) << 16);
          v[k].z = f32_to_bf16_bits(b.x) | (f32_to_bf16_bits(b.y) << 16);
          v[k].w = f32_to_bf16_bits(b.z) | (f32_to_bf16_bits(b.w) << 16);
        } else {
          v[k].x = f32_to_f16_bits(a.x) | (f32_to_f16_bits(a.y) << 16);
          v[k].y = f32_to_f16_bits(a.z) | (f32_to_f16_bits(a.w) << 16);
          v[k].z = f32_to_f16_bits(b.x) | (f32_to_f16_bits(b.y) << 16);
          v[k].w = f32_to_f16_bits(b.z) | (f32_to_f16_bits(b.w) << 16);
        }
      }
    }
  }

  // |x| as raw 15-bit magnitudes: integer order equals float order, and any
  // NaN pattern exceeds infinity, so a NaN in the tile surfaces as a NaN amax.
  uint32_t m = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    m = pk_max_u16(m, v[k].x & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].y & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].z & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].w & 0x7FFF7FFFu);
  }
  const uint32_t lo = m & 0xFFFFu, hi = m >> 16;
  m = block_max_u32(lo > hi ? lo : hi, lds);

  constexpr bool kHalf = KIND == FSH_SRC_F16 || KIND == FSH_SRC_F32_AS_F16;
  float scale, recip;
  tile_scale(kHalf ? f16_bits_to_f32(m) : bf16_bits_to_f32(m), eps, scale, recip);
  if (tid == 0)
    *reinterpret_cast<float*>(payload + ch.scale_offset + 4 * (tr * ch.tiles_c + tc)) = recip;

#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t row = row_base + 16 * k;
    if (col_ok && row < ch.rows) {
      const uint32_t d[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e0 = (kHalf ? f16_bits_to_f32(d[j] & 0xFFFFu) : u32_as_f32(d[j] << 16)) * scale;
        const float e1 = (kHalf ? f16_bits_to_f32(d[j] >> 16) : u32_as_f32(d[j] & 0xFFFF0000u)) * scale;
        w[j >> 1] = cvt2_fp8(e0, e1, w[j >> 1], (j & 1) != 0);
      }
      store_stream_u32x2(payload + ch.qdata_offset + row * ch.in_dim + col, w[0], w[1]);
    }
  }
}

// fp32 source quantized as fp32: 64 floats per thread.
__device__ __forceinline__ void quant_tile128_f32(const QuantChunkDev& ch, int64_t tr, int64_t tc,
                                                  uint8_t* payload, float eps, uint32_t* lds) {
  const int tid = threadIdx.x;
  const int g = tid & 15;
  const int r0 = tid >> 4;
  const int64_t row_base = tr * 128 + r0;
  const int64_t col = tc * 128 + g * 8;
  const bool col_ok = col < ch.in_dim;

  f32x4 v[8][2];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t row = row_base + 16 * k;
    v[k][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    v[k][1] = v[k][0];
    if (col_ok && row < ch.rows) {
      const uint8_t* p = ch.src + (row * ch.src_row_stride + col) * 4;
      v[k][0] = load_stream_f32x4(p);
      v[k][1] = load_stream_f32x4(p + 16);
    }
  }
  uint32_t m = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float e[4] = {v[k][h].x, v[k][h].y, v[k][h].z, v[k][h].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t mag = f32_as_u32(e[j]) & 0x7FFFFFFFu;
        m = mag > m ? mag : m;
      }
    }
  m = block_max_u32(m, lds);

  float scale, recip;
  tile_scale(u32_as_f32(m), eps, scale, recip);
  if (tid == 0)
    *reinterpret_cast<float*>(payload + ch.scale_offset + 4 * (tr * ch.tiles_c + tc)) = recip;

#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t row = row_base + 16 * k;
    if (col_ok && row < ch.rows) {
      uint32_t w[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint32_t packed = 0;
        packed = cvt2_fp8(v[k][h].x * scale, v[k][h].y * scale, packed, false);
        packed = cvt2_fp8(v[k][h].z * scale, v[k][h].w * scale, packed, true);
        w[h] = packed;
      }
      store_stream_u32x2(payload + ch.qdata_offset + row * ch.in_dim + col, w[0], w[1]);
    }
  }
}

// ------------------------------------------------------------- scalar path
// Any block size, any alignment: two passes over the tile with element loads.
__device__ __forceinline__ float load_as_quant_dtype(const QuantChunkDev& ch, int64_t row, int64_t col) {
  const int64_t idx = row * ch.src_row_stride + col;
  if (ch.src_kind == FSH_SRC_BF16)
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(ch.src)[idx]);
  if (ch.src_kind == FSH_SRC_F16) return static_cast<float>(reinterpret_cast<const _Float16*>(ch.src)[idx]);
  const float f = reinterpret_cast<const float*>(ch.src)[idx];
  if (ch.src_kind == FSH_SRC_F32_AS_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(f));
  if (ch.src_kind == FSH_SRC_F32_AS_F16) return f32_round_to_f16(f);
  return f;
}

__device__ void quant_tile_scalar(const QuantChunkDev& ch, int64_t tr, int64_t tc, int block,
                                  uint8_t* payload, float eps, uint32_t* lds) {
  const int tid = threadIdx.x;
  const int64_t row0 = tr * block, col0 = tc * block;
  const int64_t nrows = (ch.rows - row0) < block ? (ch.rows - row0) : block;
  const int64_t ncols = (ch.in_dim - col0) < block ? (ch.in_dim - col0) : block;
  const int64_t n = nrows * ncols;
  uint32_t m = 0;
  for (int64_t i = tid; i < n; i += kThreads) {
    const uint32_t mag = f32_as_u32(load_as_quant_dtype(ch, row0 + i / ncols, col0 + i % ncols)) & 0x7FFFFFFFu;
    m = mag > m ? mag : m;
  }
  m = block_max_u32(m, lds);
  float scale, recip;
  tile_scale(u32_as_f32(m), eps, scale, recip);
  if (tid == 0)
    *reinterpret_cast<float*>(payload + ch.scale_offset + 4 * (tr * ch.tiles_c + tc)) = recip;
  for (int64_t i = tid; i < n; i += kThreads) {
    const int64_t row = row0 + i / ncols, col = col0 + i % ncols;
    const float p = load_as_quant_dtype(ch, row, col) * scale;
    payload[ch.qdata_offset + row * ch.in_dim + col] = static_cast<uint8_t>(cvt2_fp8(p, 0.0f, 0u, false) & 0xFFu);
  }
}

// Zeroes this pad workgroup's 64 KiB slice of the two pad ranges laid end to end.
__device__ __forceinline__ void zero_pad_slice(uint8_t* payload, const int64_t (&zero_begin)[2],
                                               const int64_t (&zero_len)[2], int64_t slice) {
  const int64_t begin = slice * kZeroChunk;
  const int64_t end = begin + kZeroChunk;
  int64_t base = 0;
#pragma unroll
  for (int z = 0; z < 2; ++z) {
    const int64_t lo = begin > base ? begin : base;
    const int64_t limit = base + zero_len[z];
    const int64_t hi = end < limit ? end : limit;
    if (lo < hi) zero_bytes(payload + zero_begin[z] + (lo - base), hi - lo, threadIdx.x, kThreads);
    base = limit;
  }
}

// General kernel: any mix of source kinds, block sizes and alignments.
__global__ __launch_bounds__(kThreads) void quantize_pack_kernel(const QuantParams prm) {
  __shared__ uint32_t lds[4];
  const int64_t bid = blockIdx.x;
  if (bid >= prm.total_tiles) {
    zero_pad_slice(prm.payload, prm.zero_begin, prm.zero_len, bid - prm.total_tiles);
    return;
  }
  int c = 0;
  while (c + 1 < prm.nchunks && bid >= prm.chunks[c + 1].tile_begin) ++c;
  const QuantChunkDev& ch = prm.chunks[c];
  const int64_t t = bid - ch.tile_begin;
  const int64_t tr = t / ch.tiles_c;
  const int64_t tc = t - tr * ch.tiles_c;
  const float eps = prm.eps[ch.src_kind];
  if (ch.fast) {
    if (ch.src_kind == FSH_SRC_BF16)
      quant_tile128_bf16<FSH_SRC_BF16>(ch, tr, tc, prm.payload, eps, lds);
    else if (ch.src_kind == FSH_SRC_F32_AS_BF16)
      quant_tile128_bf16<FSH_SRC_F32_AS_BF16>(ch, tr, tc, prm.payload, eps, lds);
    else if (ch.src_kind == FSH_SRC_F16)
      quant_tile128_bf16<FSH_SRC_F16>(ch, tr, tc, prm.payload, eps, lds);
    else if (ch.src_kind == FSH_SRC_F32_AS_F16)
      quant_tile128_bf16<FSH_SRC_F32_AS_F16>(ch, tr, tc, prm.payload, eps, lds);
    else
      quant_tile128_f32(ch, tr, tc, prm.payload, eps, lds);
  } else {
    quant_tile_scalar(ch, tr, tc, prm.block, prm.payload, eps, lds);
  }
}

// ------------------------------------------------ bf16 kernel (the hot one)
// Every chunk is a 16-byte-friendly bf16 shard with 128x128 tiles.  All of a
// rank share's ~1700 workgroups are resident at once and each runs exactly
// once, so whatever precedes a workgroup's first load is added to the whole
// launch: the chunk is found with independent scalar loads (one compare per
// table entry, no dependent chain), its descriptor arrives in one more round
// trip with pointers already resolved, tile indices are 32-bit, and interior
// tiles skip every bounds test.  The tile itself is 32 dwords per thread
// (under 64 VGPRs, 8 workgroups per compute unit).
struct FastChunk {
  const uint8_t* src;     // first element of the chunk
  uint8_t* qdst;          // payload + qdata_offset
  float* scales;          // payload + scale_offset
  int64_t src_row_bytes;
  int32_t rows;
  int32_t in_dim;
  int32_t tiles_c;
  int32_t tile_begin;
};

// Entry `nchunks` of both tables stands for the pad workgroups that follow
// the tiles: its first "tile" is the total tile count.  N is 8 for the usual
// rank share (a handful of parameters: the whole lookup header is then one
// 32-byte scalar load) and FSH_MAX_QUANT_CHUNKS otherwise.
template <int N>
struct QuantFastParams {
  int32_t next_begin[N];  // first tile of chunk i + 1; INT32_MAX past the pad entry
  int32_t nchunks;
  float eps;
  FastChunk chunks[N + 1];
  uint8_t* payload;
  int64_t zero_begin[2];
  int64_t zero_len[2];
};

// Two floats -> two bf16 in one word (low half first), round to nearest even:
// one v_cvt_pk_bf16_f32.  Finite values and infinities get the bits of
// f32_to_bf16_bits; a NaN keeps its sign and payload (see canonical_nan_pair).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t round_pair_to_bf16(float lo, float hi) {
  const f32x2_t pair = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
}
// Each bf16 half that is a NaN becomes 0x7FC0, what f32_to_bf16_bits gives.
__device__ __forceinline__ uint32_t canonical_nan_pair(uint32_t w) {
  if ((w & 0x7FFFu) > 0x7F80u) w = (w & 0xFFFF0000u) | 0x7FC0u;
  if ((w & 0x7FFF0000u) > 0x7F800000u) w = (w & 0xFFFFu) | 0x7FC00000u;
  return w;
}

// F32: the shard is an fp32 master; every element is rounded to bf16 as it is
// loaded (two 16-byte loads per eight elements), four of a thread's eight tile
// rows at a time: 79 registers and six workgroups per compute unit instead of
// 91 and five with all sixteen loads in flight (forced to 72 or 64 registers
// the compiler spills and the launch is 4 % slower).
template <bool FULL, bool F32>
__device__ __forceinline__ void quant_tile128_fast(const FastChunk& ch, uint32_t tr, uint32_t tc, float eps,
                                                   uint32_t* lds) {
  const uint32_t tid = threadIdx.x;
  const uint32_t g = tid & 15;
  const uint32_t row0 = tr * 128u + (tid >> 4);
  const uint32_t col = tc * 128u + g * 8u;
  const bool col_ok = FULL || col < static_cast<uint32_t>(ch.in_dim);
  const uint32_t rows = static_cast<uint32_t>(ch.rows);
  const int64_t src_row_bytes = ch.src_row_bytes;
  const int64_t dst_row_bytes = ch.in_dim;
  const uint8_t* sp = ch.src + static_cast<int64_t>(row0) * src_row_bytes + static_cast<int64_t>(col) * (F32 ? 4 : 2);
  uint8_t* dp = ch.qdst + static_cast<int64_t>(row0) * dst_row_bytes + col;
  float* scale_slot = ch.scales + static_cast<int64_t>(tr) * ch.tiles_c + tc;

  u32x4 v[8];
  if (!F32) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (FULL) {
        v[k] = load_stream_u32x4(sp + 16 * k * src_row_bytes);
      } else {
        v[k] = u32x4{0, 0, 0, 0};
        if (col_ok && row0 + 16u * k < rows) v[k] = load_stream_u32x4(sp + 16 * k * src_row_bytes);
      }
    }
  } else {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      f32x4 a[4], b[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = 4 * half + j;
        a[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        b[j] = a[j];
        if (FULL || (col_ok && row0 + 16u * k < rows)) {
          a[j] = load_stream_f32x4(sp + 16 * k * src_row_bytes);
          b[j] = load_stream_f32x4(sp + 16 * k * src_row_bytes + 16);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = 4 * half + j;
        v[k].x = round_pair_to_bf16(a[j].x, a[j].y);
        v[k].y = round_pair_to_bf16(a[j].z, a[j].w);
        v[k].z = round_pair_to_bf16(b[j].x, b[j].y);
        v[k].w = round_pair_to_bf16(b[j].z, b[j].w);
      }
      // The second half's loads stay behind the first half's conversions
      // (the scheduler by itself hoists them above).
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // |x| as raw 15-bit magnitudes: integer order equals float order, and any
  // NaN pattern exceeds infinity, so a NaN in the tile surfaces as a NaN amax.
  uint32_t m = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    m = pk_max_u16(m, v[k].x & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].y & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].z & 0x7FFF7FFFu);
    m = pk_max_u16(m, v[k].w & 0x7FFF7FFFu);
  }
  uint32_t lo = m & 0xFFFFu, hi = m >> 16;
  if (F32 && (lo > hi ? lo : hi) > 0x7F80u) {
    // This thread rounded a NaN.  The hardware conversion keeps its sign and
    // payload; the quantization's NaN is the canonical one (0x7FC0), whose
    // bits reach the stored scale and the sign of the tile's bytes.
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      v[k].x = canonical_nan_pair(v[k].x);
      v[k].y = canonical_nan_pair(v[k].y);
      v[k].z = canonical_nan_pair(v[k].z);
      v[k].w = canonical_nan_pair(v[k].w);
    }
    lo = hi = 0x7FC0u;
  }
  m = block_max_u32(lo > hi ? lo : hi, lds);

  float scale, recip;
  tile_scale(bf16_bits_to_f32(m), eps, scale, recip);
  if (tid == 0) *scale_slot = recip;

#pragma unroll
  for (int k = 0; k < 8; ++k) {
    if (FULL || (col_ok && row0 + 16u * k < rows)) {
      const uint32_t d[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e0 = u32_as_f32(d[j] << 16) * scale;
        const float e1 = u32_as_f32(d[j] & 0xFFFF0000u) * scale;
        w[j >> 1] = cvt2_fp8(e0, e1, w[j >> 1], (j & 1) != 0);
      }
      store_stream_u32x2(dp + 16 * k * dst_row_bytes, w[0], w[1]);
    }
  }
}

template <int N>
__global__ __launch_bounds__(kThreads) void quantize_pack_bf16_kernel(const QuantFastParams<N> prm) {
  __shared__ uint32_t lds[4];
  const int32_t bid = static_cast<int32_t>(blockIdx.x);
  int c = 0;
#pragma unroll
  for (int i = 0; i < N; ++i) c += bid >= prm.next_begin[i] ? 1 : 0;
  if (c >= prm.nchunks) {
    zero_pad_slice(prm.payload, prm.zero_begin, prm.zero_len, bid - prm.chunks[c].tile_begin);
    return;
  }
  const FastChunk ch = prm.chunks[c];
  const uint32_t t = static_cast<uint32_t>(bid - ch.tile_begin);
  const uint32_t tr = t / static_cast<uint32_t>(ch.tiles_c);
  const uint32_t tc = t - tr * static_cast<uint32_t>(ch.tiles_c);
  const bool full = (tr + 1) * 128u <= static_cast<uint32_t>(ch.rows) &&
                    (tc + 1) * 128u <= static_cast<uint32_t>(ch.in_dim);
  if (full)
    quant_tile128_fast<true, false>(ch, tr, tc, prm.eps, lds);
  else
    quant_tile128_fast<false, false>(ch, tr, tc, prm.eps, lds);
}

// The same launch for fp32 master shards quantized as bf16 (the parameter
// dtype of a mixed-precision policy): 4 B read + 1 B written per element.
template <int N>
__global__ __launch_bounds__(kThreads) void quantize_pack_f32_master_kernel(const QuantFastParams<N> prm) {
  __shared__ uint32_t lds[4];
  const int32_t bid = static_cast<int32_t>(blockIdx.x);
  int c = 0;
#pragma unroll
  for (int i = 0; i < N; ++i) c += bid >= prm.next_begin[i] ? 1 : 0;
  if (c >= prm.nchunks) {
    zero_pad_slice(prm.payload, prm.zero_begin, prm.zero_len, bid - prm.chunks[c].tile_begin);
    return;
  }
  const FastChunk ch = prm.chunks[c];
  const uint32_t t = static_cast<uint32_t>(bid - ch.tile_begin);
  const uint32_t tr = t / static_cast<uint32_t>(ch.tiles_c);
  const uint32_t tc = t - tr * static_cast<uint32_t>(ch.tiles_c);
  const bool full = (tr + 1) * 128u <= static_cast<uint32_t>(ch.rows) &&
                    (tc + 1) * 128u <= static_cast<uint32_t>(ch.in_dim);
  if (full)
    quant_tile128_fast<true, true>(ch, tr, tc, prm.eps, lds);
  else
    quant_tile128_fast<false, true>(ch, tr, tc, prm.eps, lds);
}

template <int N, bool F32>
void launch_bf16_kernel(const QuantParams& prm, int64_t tiles, int64_t grid, hipStream_t stream) {
  QuantFastParams<N> fast;
  memset(&fast, 0, sizeof(fast));
  const int nchunks = prm.nchunks;
  for (int i = 0; i < N; ++i) fast.next_begin[i] = INT32_MAX;
  for (int i = 0; i < nchunks; ++i) {
    const QuantChunkDev& in = prm.chunks[i];
    FastChunk& out = fast.chunks[i];
    out.src = in.src;
    out.qdst = prm.payload + in.qdata_offset;
    out.scales = reinterpret_cast<float*>(prm.payload + in.scale_offset);
    out.src_row_bytes = in.src_row_stride * (F32 ? 4 : 2);
    out.rows = static_cast<int32_t>(in.rows);
    out.in_dim = static_cast<int32_t>(in.in_dim);
    out.tiles_c = in.tiles_c;
    out.tile_begin = static_cast<int32_t>(in.tile_begin);
    if (i > 0) fast.next_begin[i - 1] = out.tile_begin;
  }
  fast.chunks[nchunks].tile_begin = static_cast<int32_t>(tiles);
  fast.chunks[nchunks].tiles_c = 1;
  if (nchunks > 0) fast.next_begin[nchunks - 1] = static_cast<int32_t>(tiles);
  fast.payload = prm.payload;
  for (int z = 0; z < 2; ++z) {
    fast.zero_begin[z] = prm.zero_begin[z];
    fast.zero_len[z] = prm.zero_len[z];
  }
  fast.eps = prm.eps[F32 ? FSH_SRC_F32_AS_BF16 : FSH_SRC_BF16];
  fast.nchunks = nchunks;
  if (F32)
    hipLaunchKernelGGL(quantize_pack_f32_master_kernel<N>, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0,
                       stream, fast);
  else
    hipLaunchKernelGGL(quantize_pack_bf16_kernel<N>, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0, stream,
                       fast);
}

float bf16_round_host(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  memcpy(&f, &u, 4);
  return f;
}

}  // namespace
}  // namespace fsh

// A reusable launch: the arguments of fsh_quantize_pack except the payload
// address and the stream.  More than FSH_MAX_QUANT_CHUNKS chunks become several
// launches, the first of which also zeroes the pad ranges.
struct fsh_quant_pack_plan {
  std::vector<fsh_quant_chunk> chunks;
  int64_t payload_nbytes;
  int64_t zero[4];
  int32_t block;
  int32_t eps_mode;
};

static int quantize_pack_impl(const fsh_quant_chunk* chunks, int32_t nchunks, void* payload_dev,
                              int64_t payload_nbytes, int64_t zero0_begin, int64_t zero0_end,
                              int64_t zero1_begin, int64_t zero1_end, int32_t block,
                              int32_t eps_mode, void* stream, bool launch);

FSH_API int fsh_quantize_pack(const fsh_quant_chunk* chunks, int32_t nchunks, void* payload_dev,
                              int64_t payload_nbytes, int64_t zero0_begin, int64_t zero0_end,
                              int64_t zero1_begin, int64_t zero1_end, int32_t block,
                              int32_t eps_mode, void* stream) {
  return quantize_pack_impl(chunks, nchunks, payload_dev, payload_nbytes, zero0_begin, zero0_end, zero1_begin,
                            zero1_end, block, eps_mode, stream, true);
}

FSH_API int fsh_quant_pack_plan_create(const fsh_quant_chunk* chunks, int32_t nchunks, int64_t payload_nbytes,
                                       int64_t zero0_begin, int64_t zero0_end, int64_t zero1_begin,
                                       int64_t zero1_end, int32_t block, int32_t eps_mode, void** plan_out) {
  using namespace fsh;
  if (plan_out == nullptr) return fail(FSH_EINVAL, "fsh_quant_pack_plan_create: null plan_out");
  *plan_out = nullptr;
  if (nchunks < 0 || (nchunks > 0 && chunks == nullptr))
    return fail(FSH_EINVAL, "fsh_quant_pack_plan_create: bad chunk table (%d chunks)", nchunks);
  // Every launch of the plan is checked now, against a stand-in payload
  // address with the alignment a launch will ask for; nothing is queued.
  void* const probe = reinterpret_cast<void*>(static_cast<uintptr_t>(4096));
  int32_t first = 0;
  do {
    const int32_t count = std::min<int32_t>(nchunks - first, FSH_MAX_QUANT_CHUNKS);
    const bool lead = first == 0;
    const int status = quantize_pack_impl(chunks + first, count, payload_nbytes > 0 ? probe : nullptr, payload_nbytes,
                                          lead ? zero0_begin : 0, lead ? zero0_end : 0, lead ? zero1_begin : 0,
                                          lead ? zero1_end : 0, block, eps_mode, nullptr, false);
    if (status != FSH_OK) return status;
    first += count;
  } while (first < nchunks);
  fsh_quant_pack_plan* plan = new (std::nothrow) fsh_quant_pack_plan();
  if (plan == nullptr) return fail(FSH_EINVAL, "fsh_quant_pack_plan_create: out of host memory");
  plan->chunks.assign(chunks, chunks + nchunks);
  plan->payload_nbytes = payload_nbytes;
  plan->zero[0] = zero0_begin, plan->zero[1] = zero0_end, plan->zero[2] = zero1_begin, plan->zero[3] = zero1_end;
  plan->block = block;
  plan->eps_mode = eps_mode;
  *plan_out = plan;
  return FSH_OK;
}

FSH_API int fsh_quant_pack_plan_launch(const void* plan_handle, void* payload_dev, void* stream) {
  using namespace fsh;
  if (plan_handle == nullptr) return fail(FSH_EINVAL, "fsh_quant_pack_plan_launch: null plan");
  const fsh_quant_pack_plan& plan = *static_cast<const fsh_quant_pack_plan*>(plan_handle);
  const int32_t nchunks = static_cast<int32_t>(plan.chunks.size());
  int32_t first = 0;
  do {
    const int32_t count = std::min<int32_t>(nchunks - first, FSH_MAX_QUANT_CHUNKS);
    const bool lead = first == 0;
    const int status =
        quantize_pack_impl(plan.chunks.data() + first, count, payload_dev, plan.payload_nbytes,
                           lead ? plan.zero[0] : 0, lead ? plan.zero[1] : 0, lead ? plan.zero[2] : 0,
                           lead ? plan.zero[3] : 0, plan.block, plan.eps_mode, stream, true);
    if (status != FSH_OK) return status;
    first += count;
  } while (first < nchunks);
  return FSH_OK;
}

FSH_API void fsh_quant_pack_plan_destroy(void* plan_handle) {
  delete static_cast<fsh_quant_pack_plan*>(plan_handle);
}

static int quantize_pack_impl(const fsh_quant_chunk* chunks, int32_t nchunks, void* payload_dev,
                              int64_t payload_nbytes, int64_t zero0_begin, int64_t zero0_end,
                              int64_t zero1_begin, int64_t zero1_end, int32_t block,
                              int32_t eps_mode, void* stream, bool launch) {
  using namespace fsh;
  if (nchunks < 0 || nchunks > FSH_MAX_QUANT_CHUNKS)
    return fail(FSH_EINVAL, "fsh_quantize_pack: nchunks %d outside [0, %d]", nchunks, FSH_MAX_QUANT_CHUNKS);
  if (nchunks > 0 && chunks == nullptr) return fail(FSH_EINVAL, "fsh_quantize_pack: null chunk table");
  if (block <= 0) return fail(FSH_EINVAL, "fsh_quantize_pack: block must be positive, got %d", block);
  if (eps_mode != FSH_EPS_INPUT_DTYPE && eps_mode != FSH_EPS_FP32)
    return fail(FSH_EINVAL, "fsh_quantize_pack: unknown eps_mode %d", eps_mode);
  if (payload_nbytes < 0 || (payload_nbytes > 0 && payload_dev == nullptr))
    return fail(FSH_EINVAL, "fsh_quantize_pack: bad payload");
  if (!aligned(payload_dev, 16)) return fail(FSH_EINVAL, "fsh_quantize_pack: payload must be 16-byte aligned");
  const int64_t zb[2] = {zero0_begin, zero1_begin}, ze[2] = {zero0_end, zero1_end};
  for (int z = 0; z < 2; ++z)
    if (zb[z] < 0 || ze[z] < zb[z] || ze[z] > payload_nbytes)
      return fail(FSH_EINVAL, "fsh_quantize_pack: zero range %d [%lld, %lld) outside payload of %lld bytes", z,
                  (long long)zb[z], (long long)ze[z], (long long)payload_nbytes);

  QuantParams prm;
  memset(&prm, 0, sizeof(prm));
  prm.payload = static_cast<uint8_t*>(payload_dev);
  prm.nchunks = nchunks;
  prm.block = block;
  const float eps32 = 1e-12f;
  const float eps_bf16 = eps_mode == FSH_EPS_FP32 ? eps32 : bf16_round_host(eps32);
  prm.eps[FSH_SRC_BF16] = eps_bf16;
  prm.eps[FSH_SRC_F32] = eps32;
  prm.eps[FSH_SRC_F32_AS_BF16] = eps_bf16;
  // 1e-12 is below fp16's smallest subnormal (6e-8): in the input dtype the
  // floor is 0, and an all-zero tile gets scale inf, reciprocal 0 and NaN
  // bytes, as the reference's arithmetic gives.
  prm.eps[FSH_SRC_F16] = prm.eps[FSH_SRC_F32_AS_F16] = eps_mode == FSH_EPS_FP32 ? eps32 : 0.0f;

  int64_t tiles = 0;
  bool all_bf16_fast = true, all_f32_master_fast = true;
  for (int i = 0; i < nchunks; ++i) {
    const fsh_quant_chunk& in = chunks[i];
    if (in.src_dev == nullptr || in.rows <= 0 || in.in_dim <= 0 || in.src_row_stride < in.in_dim)
      return fail(FSH_EINVAL, "fsh_quantize_pack: chunk %d has bad shape (rows %lld, in_dim %lld, stride %lld)", i,
                  (long long)in.rows, (long long)in.in_dim, (long long)in.src_row_stride);
    if (in.src_kind < 0 || in.src_kind > FSH_SRC_F32_AS_F16)
      return fail(FSH_EINVAL, "fsh_quantize_pack: chunk %d has unknown src_kind %d", i, in.src_kind);
    const int64_t tiles_r = ceil_div(in.rows, block), tiles_c = ceil_div(in.in_dim, block);
    if (in.qdata_offset < 0 || in.qdata_offset + in.rows * in.in_dim > payload_nbytes)
      return fail(FSH_EINVAL, "fsh_quantize_pack: chunk %d data [%lld, +%lld) outside payload", i,
                  (long long)in.qdata_offset, (long long)(in.rows * in.in_dim));
    if (in.scale_offset < 0 || (in.scale_offset & 3) != 0 ||
        in.scale_offset + 4 * tiles_r * tiles_c > payload_nbytes)
      return fail(FSH_EINVAL, "fsh_quantize_pack: chunk %d scales at %lld misaligned or outside payload", i,
                  (long long)in.scale_offset);
    const int64_t elem = (in.src_kind == FSH_SRC_BF16 || in.src_kind == FSH_SRC_F16) ? 2 : 4;
    if (!aligned(in.src_dev, elem)) return fail(FSH_EINVAL, "fsh_quantize_pack: chunk %d source misaligned", i);
    QuantChunkDev& out = prm.chunks[i];
    out.src = static_cast<const uint8_t*>(in.src_dev);
    out.rows = in.rows;
    out.in_dim = in.in_dim;
    out.src_row_stride = in.src_row_stride;
    out.qdata_offset = in.qdata_offset;
    out.scale_offset = in.scale_offset;
    out.tile_begin = tiles;
    out.tiles_c = static_cast<int32_t>(tiles_c);
    out.src_kind = in.src_kind;
    out.fast = block == 128 && aligned(in.src_dev, 16) && (in.src_row_stride * elem) % 16 == 0 &&
               in.in_dim % 8 == 0 && in.qdata_offset % 8 == 0;
    const bool small = in.rows < (1LL << 30) && in.in_dim < (1LL << 30);
    all_bf16_fast = all_bf16_fast && out.fast && in.src_kind == FSH_SRC_BF16 && small;
    all_f32_master_fast = all_f32_master_fast && out.fast && in.src_kind == FSH_SRC_F32_AS_BF16 && small;
    tiles += tiles_r * tiles_c;
  }
  prm.total_tiles = tiles;
  int64_t zero_total = 0;
  for (int z = 0; z < 2; ++z) {
    prm.zero_begin[z] = zb[z];
    prm.zero_len[z] = ze[z] - zb[z];
    zero_total += prm.zero_len[z];
  }
  const int64_t grid = tiles + ceil_div(zero_total, kZeroChunk);
  if (grid == 0) return FSH_OK;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_quantize_pack: %lld workgroups exceed the grid limit", (long long)grid);
  if (!launch) return FSH_OK;
  if (all_bf16_fast) {
    if (nchunks < 8)
      launch_bf16_kernel<8, false>(prm, tiles, grid, static_cast<hipStream_t>(stream));
    else
      launch_bf16_kernel<FSH_MAX_QUANT_CHUNKS, false>(prm, tiles, grid, static_cast<hipStream_t>(stream));
  } else if (all_f32_master_fast && nchunks > 0) {
    if (nchunks < 8)
      launch_bf16_kernel<8, true>(prm, tiles, grid, static_cast<hipStream_t>(stream));
    else
      launch_bf16_kernel<FSH_MAX_QUANT_CHUNKS, true>(prm, tiles, grid, static_cast<hipStream_t>(stream));
  } else {
    hipLaunchKernelGGL(quantize_pack_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), prm);
  }
  return check_launch("fsh_quantize_pack");
}
