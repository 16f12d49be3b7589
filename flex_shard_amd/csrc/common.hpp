// Shared helpers of the gfx950 kernels: error reporting, launch checks, bit
// conversions, cooperative byte copy/fill with run-time vector width.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/flexshard_hip.h"

#define FSH_API extern "C" __attribute__((visibility("default")))

namespace fsh {

// Thread-local message of the last failed call.
char* error_buffer();
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

inline bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int kWave = 64;

// Native vector types (the nontemporal builtins reject HIP's struct vectors).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Streaming (nontemporal) 16/8-byte accesses: the hot kernels touch every
// byte once, so nothing is worth keeping in the caches.
__device__ __forceinline__ u32x4 load_stream_u32x4(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ f32x4 load_stream_f32x4(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
}
__device__ __forceinline__ void store_stream_u32x2(void* p, uint32_t a, uint32_t b) {
  u32x2 v = {a, b};
  __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
}
__device__ __forceinline__ void store_stream_u32x4(void* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// ---------------------------------------------------------------- bit casts
__device__ __forceinline__ float u32_as_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_as_u32(float f) { return __float_as_uint(f); }

// bf16 bits (low 16 of `h`) -> float, exact.
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return u32_as_f32(h << 16); }

// float -> bf16 bits, round to nearest even, NaN -> 0x7FC0.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = f32_as_u32(f);
  uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  return (f != f) ? 0x7FC0u : r;
}

// float -> fp16 bits, round to nearest even over the whole range, subnormal
// results included, in integer arithmetic plus one fp32 add: the hardware
// conversion rounded exact ties of subnormal results away from zero (e.g.
// 690.5 x 2^-24 to 691) where torch's cast gives the even neighbour.
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  uint32_t u = f32_as_u32(f);
  const uint32_t sign = (u >> 16) & 0x8000u;
  u &= 0x7FFFFFFFu;
  uint32_t h;
  if (u >= 0x47800000u) {  // 65536 and above, infinity, NaN
    h = u > 0x7F800000u ? 0x7E00u : 0x7C00u;
  } else if (u < 0x38800000u) {  // below 2^-14: the sum's low mantissa bits are the subnormal's
    h = f32_as_u32(u32_as_f32(u) + 0.5f) - 0x3F000000u;
  } else {  // rebias the exponent, add half an ulp (to even), carry into the exponent up to infinity
    h = (u + 0xC8000FFFu + ((u >> 13) & 1u)) >> 13;
  }
  return sign | h;
}
// The fp16 value nearest to f, as a float.
// fp16 bits (low 16 of `h`) -> float, exact.
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}
__device__ __forceinline__ float f32_round_to_f16(float f) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(f32_to_f16_bits(f))));
}

// Integer max across the 64 lanes of a wavefront, result in every lane.
// Data-parallel-primitive moves: two quad permutes, two mirrors inside each
// row of 16 lanes, then two row broadcasts leave the total in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
  const uint32_t o = static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(static_cast<int>(v), static_cast<int>(v), CTRL, ROW_MASK, 0xF, false));
  return o > v ? o : v;
}
// Maximum over each row of 16 lanes, in every lane of the row.
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v) {
  v = dpp_max_u32<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_max_u32<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_max_u32<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_max_u32<0x140, 0xF>(v);  // row_mirror
  return v;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = dpp_max_u32<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_max_u32<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_max_u32<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_max_u32<0x140, 0xF>(v);  // row_mirror
  v = dpp_max_u32<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_max_u32<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// ------------------------------------------------- FP8 quantizer arithmetic
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  u16x2 va = __builtin_bit_cast(u16x2, a);
  u16x2 vb = __builtin_bit_cast(u16x2, b);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(va, vb));
}

// Two floats -> two E4M3FN bytes in the low (hi=false) or high half of `old`.
__device__ __forceinline__ uint32_t cvt2_fp8(float a, float b, uint32_t old, bool hi) {
  return hi ? static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, static_cast<int>(old), true))
            : static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, static_cast<int>(old), false));
}

// Scale pair of a tile from its amax; identical on every lane.
__device__ __forceinline__ void tile_scale(float amax, float eps, float& scale, float& recip) {
  const float floored = (amax < eps) ? eps : amax;  // NaN fails the test and stays
  scale = static_cast<float>(448.0 / static_cast<double>(floored));
  recip = 1.0f / scale;
}

// ------------------------------------------------- cooperative byte movers
// All threads of the workgroup call these with identical arguments.  The
// widest vector the relative alignment of src and dst allows is used for the
// bulk; unaligned heads and tails move as bytes.
template <typename V>
__device__ __forceinline__ void copy_bulk(const uint8_t* src, uint8_t* dst, int64_t n, int tid,
                                          int nthreads) {
  // Precondition: src and dst are congruent modulo sizeof(V).
  int64_t head = (sizeof(V) - (reinterpret_cast<uintptr_t>(dst) & (sizeof(V) - 1))) & (sizeof(V) - 1);
  if (head > n) head = n;
  for (int64_t i = tid; i < head; i += nthreads) dst[i] = src[i];
  const int64_t body = (n - head) / static_cast<int64_t>(sizeof(V));
  const V* s = reinterpret_cast<const V*>(src + head);
  V* d = reinterpret_cast<V*>(dst + head);
  if (sizeof(V) == 16) {
    // The 16-byte body streams: a nontemporal load with a plain store measured
    // 13 % faster on a 436 MB copy than plain/plain, and than either other mix.
    for (int64_t i = tid; i < body; i += nthreads)
      reinterpret_cast<u32x4*>(d)[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s) + i);
  } else {
    for (int64_t i = tid; i < body; i += nthreads) d[i] = s[i];
  }
  const int64_t done = head + body * static_cast<int64_t>(sizeof(V));
  for (int64_t i = done + tid; i < n; i += nthreads) dst[i] = src[i];
}

__device__ __forceinline__ void copy_bytes(const uint8_t* src, uint8_t* dst, int64_t n, int tid,
                                           int nthreads) {
  const uintptr_t rel = reinterpret_cast<uintptr_t>(src) ^ reinterpret_cast<uintptr_t>(dst);
  if ((rel & 15) == 0)
    copy_bulk<uint4>(src, dst, n, tid, nthreads);
  else if ((rel & 7) == 0)
    copy_bulk<uint2>(src, dst, n, tid, nthreads);
  else if ((rel & 3) == 0)
    copy_bulk<uint32_t>(src, dst, n, tid, nthreads);
  else if ((rel & 1) == 0)
    copy_bulk<uint16_t>(src, dst, n, tid, nthreads);
  else
    for (int64_t i = tid; i < n; i += nthreads) dst[i] = src[i];
}

__device__ __forceinline__ void zero_bytes(uint8_t* dst, int64_t n, int tid, int nthreads) {
  int64_t head = (16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15;
  if (head > n) head = n;
  for (int64_t i = tid; i < head; i += nthreads) dst[i] = 0;
  const int64_t body = (n - head) / 16;
  uint4* d = reinterpret_cast<uint4*>(dst + head);
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (int64_t i = tid; i < body; i += nthreads) d[i] = z;
  for (int64_t i = head + body * 16 + tid; i < n; i += nthreads) dst[i] = 0;
}

}  // namespace fsh
