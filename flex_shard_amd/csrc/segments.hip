// Segment copy / zero / cast-pack over device descriptor tables.
//
// Each kernel takes the same three (or four) int64 device arrays the Triton
// kernels they replace take.  The grid is (segment, slice): a slice is
// kSliceBytes of one segment, copied by 256 threads with the widest vector the
// relative alignment of source and destination allows (16-byte in the common
// case, falling back to 8/4/2/1-byte units, so rank rows at odd byte offsets
// work too).
#include "common.hpp"

namespace fsh {
namespace {

constexpr int kThreads = 256;
constexpr int64_t kSliceBytes = 16384;  // 4 x 16 B per thread

__global__ __launch_bounds__(kThreads) void copy_segments_kernel(
    const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, const int64_t* __restrict__ src_offsets,
    const int64_t* __restrict__ numels, const int64_t* __restrict__ dst_offsets, int64_t slices_per_segment,
    int64_t unit) {
  const int64_t seg = blockIdx.x / slices_per_segment;
  const int64_t slice = blockIdx.x - seg * slices_per_segment;
  const int64_t nbytes = numels[seg] * unit;
  const int64_t begin = slice * kSliceBytes;
  if (begin >= nbytes) return;
  const int64_t len = (nbytes - begin) < kSliceBytes ? (nbytes - begin) : kSliceBytes;
  copy_bytes(src + src_offsets[seg] * unit + begin, dst + dst_offsets[seg] * unit + begin, len, threadIdx.x,
             kThreads);
}

__global__ __launch_bounds__(kThreads) void zero_segments_kernel(uint8_t* __restrict__ dst,
                                                                const int64_t* __restrict__ numels,
                                                                const int64_t* __restrict__ dst_offsets,
                                                                int64_t slices_per_segment, int64_t unit) {
  const int64_t seg = blockIdx.x / slices_per_segment;
  const int64_t slice = blockIdx.x - seg * slices_per_segment;
  const int64_t nbytes = numels[seg] * unit;
  const int64_t begin = slice * kSliceBytes;
  if (begin >= nbytes) return;
  const int64_t len = (nbytes - begin) < kSliceBytes ? (nbytes - begin) : kSliceBytes;
  zero_bytes(dst + dst_offsets[seg] * unit + begin, len, threadIdx.x, kThreads);
}

constexpr int64_t kPackSliceElems = 2048;  // one 8-element group per thread (larger slices measured slower)

template <typename SRC, typename DST>
__device__ __forceinline__ DST cast_elem(SRC v);
template <>
__device__ __forceinline__ float cast_elem<float, float>(float v) { return v; }
template <>
__device__ __forceinline__ uint16_t cast_elem<uint16_t, uint16_t>(uint16_t v) { return v; }
template <>
__device__ __forceinline__ float cast_elem<uint16_t, float>(uint16_t v) { return bf16_bits_to_f32(v); }
template <>
__device__ __forceinline__ uint16_t cast_elem<float, uint16_t>(float v) {
  return static_cast<uint16_t>(f32_to_bf16_bits(v));
}

// Eight consecutive elements, both pointers 16-byte aligned.
__device__ __forceinline__ void cast_group_of_8(const uint16_t* src, float* dst) {
  const u32x4 v = load_stream_u32x4(src);
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
  f32x4 lo, hi;
  lo.x = u32_as_f32(d[0] << 16); lo.y = u32_as_f32(d[0] & 0xFFFF0000u);
  lo.z = u32_as_f32(d[1] << 16); lo.w = u32_as_f32(d[1] & 0xFFFF0000u);
  hi.x = u32_as_f32(d[2] << 16); hi.y = u32_as_f32(d[2] & 0xFFFF0000u);
  hi.z = u32_as_f32(d[3] << 16); hi.w = u32_as_f32(d[3] & 0xFFFF0000u);
  reinterpret_cast<f32x4*>(dst)[0] = lo;
  reinterpret_cast<f32x4*>(dst)[1] = hi;
}
__device__ __forceinline__ void cast_group_of_8(const float* src, uint16_t* dst) {
  const f32x4 a = load_stream_f32x4(src), b = load_stream_f32x4(src + 4);
  u32x4 o;
  o.x = f32_to_bf16_bits(a.x) | (f32_to_bf16_bits(a.y) << 16);
  o.y = f32_to_bf16_bits(a.z) | (f32_to_bf16_bits(a.w) << 16);
  o.z = f32_to_bf16_bits(b.x) | (f32_to_bf16_bits(b.y) << 16);
  o.w = f32_to_bf16_bits(b.z) | (f32_to_bf16_bits(b.w) << 16);
  *reinterpret_cast<u32x4*>(dst) = o;
}
// Same-type pairs never reach the casting branch; these keep it compilable.
__device__ __forceinline__ void cast_group_of_8(const float*, float*) {}
__device__ __forceinline__ void cast_group_of_8(const uint16_t*, uint16_t*) {}

// Multi-input gather with cast.  A negative tensor index marks a zero-fill
// segment.  Same-dtype segments move as bytes with the widest legal vector;
// casting segments convert element by element (coalesced across the wave).
template <typename SRC, typename DST>
__global__ __launch_bounds__(kThreads) void pack_segments_kernel(
    const int64_t* __restrict__ input_ptrs, const int64_t* __restrict__ tensor_indices,
    const int64_t* __restrict__ src_offsets, const int64_t* __restrict__ numels,
    const int64_t* __restrict__ dst_offsets, DST* __restrict__ out, int64_t slices_per_segment) {
  const int64_t seg = blockIdx.x / slices_per_segment;
  const int64_t slice = blockIdx.x - seg * slices_per_segment;
  const int64_t n = numels[seg];
  const int64_t begin = slice * kPackSliceElems;
  if (begin >= n) return;
  const int64_t len = (n - begin) < kPackSliceElems ? (n - begin) : kPackSliceElems;
  DST* dst = out + dst_offsets[seg] + begin;
  const int64_t ti = tensor_indices[seg];
  if (ti < 0) {
    zero_bytes(reinterpret_cast<uint8_t*>(dst), len * static_cast<int64_t>(sizeof(DST)), threadIdx.x, kThreads);
    return;
  }
  const SRC* src = reinterpret_cast<const SRC*>(static_cast<uintptr_t>(input_ptrs[ti])) + src_offsets[seg] + begin;
  if (sizeof(SRC) == sizeof(DST)) {
    copy_bytes(reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst),
               len * static_cast<int64_t>(sizeof(DST)), threadIdx.x, kThreads);
  } else {
    // Eight elements per thread and step when both sides start on a 16-byte
    // boundary (16 bytes of bf16 against 32 of fp32); the rest, and slices
    // that do not, go element by element.
    int64_t done = 0;
    if (((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0) {
      const int64_t groups = len / 8;
      for (int64_t g = threadIdx.x; g < groups; g += kThreads) cast_group_of_8(src + 8 * g, dst + 8 * g);
      done = groups * 8;
    }
    for (int64_t i = done + threadIdx.x; i < len; i += kThreads) dst[i] = cast_elem<SRC, DST>(src[i]);
  }
}

int check_unit(const char* who, int32_t unit) {
  if (unit != 1 && unit != 2 && unit != 4 && unit != 8 && unit != 16)
    return fail(FSH_EINVAL, "%s: unit_nbytes must be 1, 2, 4, 8 or 16, got %d", who, unit);
  return FSH_OK;
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_copy_segments(const void* src_dev, void* dst_dev, const int64_t* src_offsets_dev,
                              const int64_t* numels_dev, const int64_t* dst_offsets_dev,
                              int64_t nsegments, int64_t max_segment_numel, int32_t unit_nbytes,
                              void* stream) {
  using namespace fsh;
  if (int rc = check_unit("fsh_copy_segments", unit_nbytes)) return rc;
  if (nsegments < 0 || max_segment_numel < 0) return fail(FSH_EINVAL, "fsh_copy_segments: negative size");
  if (nsegments == 0 || max_segment_numel == 0) return FSH_OK;
  if (!src_dev || !dst_dev || !src_offsets_dev || !numels_dev || !dst_offsets_dev)
    return fail(FSH_EINVAL, "fsh_copy_segments: null pointer");
  if (!aligned(src_dev, unit_nbytes) || !aligned(dst_dev, unit_nbytes))
    return fail(FSH_EINVAL, "fsh_copy_segments: base pointers must be aligned to unit_nbytes=%d", unit_nbytes);
  const int64_t slices = ceil_div(max_segment_numel * unit_nbytes, kSliceBytes);
  const int64_t grid = nsegments * slices;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_copy_segments: %lld workgroups exceed the grid limit", (long long)grid);
  hipLaunchKernelGGL(copy_segments_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(src_dev),
                     static_cast<uint8_t*>(dst_dev), src_offsets_dev, numels_dev, dst_offsets_dev, slices,
                     static_cast<int64_t>(unit_nbytes));
  return check_launch("fsh_copy_segments");
}

FSH_API int fsh_zero_segments(void* dst_dev, const int64_t* numels_dev, const int64_t* dst_offsets_dev,
                              int64_t nsegments, int64_t max_segment_numel, int32_t unit_nbytes,
                              void* stream) {
  using namespace fsh;
  if (int rc = check_unit("fsh_zero_segments", unit_nbytes)) return rc;
  if (nsegments < 0 || max_segment_numel < 0) return fail(FSH_EINVAL, "fsh_zero_segments: negative size");
  if (nsegments == 0 || max_segment_numel == 0) return FSH_OK;
  if (!dst_dev || !numels_dev || !dst_offsets_dev) return fail(FSH_EINVAL, "fsh_zero_segments: null pointer");
  if (!aligned(dst_dev, unit_nbytes))
    return fail(FSH_EINVAL, "fsh_zero_segments: base pointer must be aligned to unit_nbytes=%d", unit_nbytes);
  const int64_t slices = ceil_div(max_segment_numel * unit_nbytes, kSliceBytes);
  const int64_t grid = nsegments * slices;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_zero_segments: %lld workgroups exceed the grid limit", (long long)grid);
  hipLaunchKernelGGL(zero_segments_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint8_t*>(dst_dev), numels_dev,
                     dst_offsets_dev, slices, static_cast<int64_t>(unit_nbytes));
  return check_launch("fsh_zero_segments");
}

FSH_API int fsh_pack_segments(const int64_t* input_ptrs_dev, const int64_t* tensor_indices_dev,
                              const int64_t* src_offsets_dev, const int64_t* numels_dev,
                              const int64_t* dst_offsets_dev, int64_t nsegments,
                              int64_t max_segment_numel, int32_t src_dtype, int32_t dst_dtype,
                              void* dst_dev, void* stream) {
  using namespace fsh;
  if (nsegments < 0 || max_segment_numel < 0) return fail(FSH_EINVAL, "fsh_pack_segments: negative size");
  if (nsegments == 0 || max_segment_numel == 0) return FSH_OK;
  if (!input_ptrs_dev || !tensor_indices_dev || !src_offsets_dev || !numels_dev || !dst_offsets_dev || !dst_dev)
    return fail(FSH_EINVAL, "fsh_pack_segments: null pointer");
  const int64_t slices = ceil_div(max_segment_numel, kPackSliceElems);
  const int64_t grid = nsegments * slices;
  if (grid > 0x7FFFFFFFLL) return fail(FSH_ENOTSUP, "fsh_pack_segments: %lld workgroups exceed the grid limit", (long long)grid);
  const dim3 g(static_cast<uint32_t>(grid)), b(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define FSH_PACK_LAUNCH(SRC, DST)                                                                      \
  hipLaunchKernelGGL((pack_segments_kernel<SRC, DST>), g, b, 0, s, input_ptrs_dev, tensor_indices_dev, \
                     src_offsets_dev, numels_dev, dst_offsets_dev, static_cast<DST*>(dst_dev), slices)
  if (src_dtype == FSH_DT_F32 && dst_dtype == FSH_DT_BF16) {
    FSH_PACK_LAUNCH(float, uint16_t);
  } else if (src_dtype == FSH_DT_BF16 && dst_dtype == FSH_DT_F32) {
    FSH_PACK_LAUNCH(uint16_t, float);
  } else if (src_dtype == FSH_DT_F32 && dst_dtype == FSH_DT_F32) {
    FSH_PACK_LAUNCH(float, float);
  } else if (src_dtype == FSH_DT_BF16 && dst_dtype == FSH_DT_BF16) {
    FSH_PACK_LAUNCH(uint16_t, uint16_t);
  } else {
    return fail(FSH_EINVAL, "fsh_pack_segments: unsupported dtype pair (%d -> %d)", src_dtype, dst_dtype);
  }
#undef FSH_PACK_LAUNCH
  return check_launch("fsh_pack_segments");
}
