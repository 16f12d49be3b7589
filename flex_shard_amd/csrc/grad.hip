// Gradient path and Muon elementwise kernels: fp32 accumulation of bf16
// microbatch gradients, fixed-order W-way fp32 reduction of one rank's range,
// momentum / Nesterov interpolation and the decoupled-weight-decay update.
// All are HBM-bound streaming kernels: 16-byte accesses, grid-stride loops
// sized to a few workgroups per compute unit.
#include "common.hpp"
#include "muon_elementwise.hpp"

namespace fsh {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxGrid = 256 * 16;  // 16 workgroups per CU on a 256-CU part

inline uint32_t grid_for(int64_t work_items) {
  int64_t g = ceil_div(work_items, kThreads);
  if (g > kMaxGrid) g = kMaxGrid;
  if (g < 1) g = 1;
  return static_cast<uint32_t>(g);
}

// acc[i] (+)= float(grad[i]); 8 elements per thread per iteration when both
// pointers are 16/32-byte friendly, scalar otherwise.
template <int GRAD_DT, bool OVERWRITE>
__global__ __launch_bounds__(kThreads) void accumulate_kernel(float* __restrict__ acc,
                                                             const uint8_t* __restrict__ grad, int64_t n,
                                                             int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gidx = tid; gidx < groups; gidx += nthreads) {
      float g[8];
      if (GRAD_DT == FSH_DT_BF16) {
        const u32x4 v = load_stream_u32x4(grad + gidx * 16);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          g[2 * j] = u32_as_f32(d[j] << 16);
          g[2 * j + 1] = u32_as_f32(d[j] & 0xFFFF0000u);
        }
      } else {
        const f32x4 a = load_stream_f32x4(grad + gidx * 32);
        const f32x4 b = load_stream_f32x4(grad + gidx * 32 + 16);
        g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w;
        g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
      }
      f32x4* out = reinterpret_cast<f32x4*>(acc + gidx * 8);
      f32x4 o0, o1;
      if (OVERWRITE) {
        o0 = f32x4{g[0], g[1], g[2], g[3]};
        o1 = f32x4{g[4], g[5], g[6], g[7]};
      } else {
        const f32x4 a0 = out[0], a1 = out[1];
        o0 = f32x4{a0.x + g[0], a0.y + g[1], a0.z + g[2], a0.w + g[3]};
        o1 = f32x4{a1.x + g[4], a1.y + g[5], a1.z + g[6], a1.w + g[7]};
      }
      out[0] = o0;
      out[1] = o1;
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads) {
    const float g = GRAD_DT == FSH_DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(grad)[i])
                                           : reinterpret_cast<const float*>(grad)[i];
    acc[i] = OVERWRITE ? g : acc[i] + g;
  }
}

// out[i] = fold_r src[r*stride + col + i], r ascending: the association
// ((x0 + x1) + x2) + ... is fixed by the loop order.
template <int MODE>
__device__ __forceinline__ float fold_term(float x, float factor) {
  return MODE == FSH_REDUCE_PREMUL ? x * factor : x;
}
template <int MODE>
__device__ __forceinline__ float fold_finish(float s, float factor) {
  if (MODE == FSH_REDUCE_POSTMUL) return s * factor;
  if (MODE == FSH_REDUCE_POSTDIV) return s / factor;
  return s;
}

template <int MODE>
__global__ __launch_bounds__(kThreads) void reduce_rows_kernel(float* __restrict__ out,
                                                              const float* __restrict__ src, int64_t stride,
                                                              int world, int64_t n, float factor, int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 4;
    for (int64_t gidx = tid; gidx < groups; gidx += nthreads) {
      f32x4 s = load_stream_f32x4(src + gidx * 4);
      s = f32x4{fold_term<MODE>(s.x, factor), fold_term<MODE>(s.y, factor), fold_term<MODE>(s.z, factor),
                fold_term<MODE>(s.w, factor)};
      for (int r = 1; r < world; ++r) {
        const f32x4 v = load_stream_f32x4(src + r * stride + gidx * 4);
        s.x = s.x + fold_term<MODE>(v.x, factor);
        s.y = s.y + fold_term<MODE>(v.y, factor);
        s.z = s.z + fold_term<MODE>(v.z, factor);
        s.w = s.w + fold_term<MODE>(v.w, factor);
      }
      s = f32x4{fold_finish<MODE>(s.x, factor), fold_finish<MODE>(s.y, factor), fold_finish<MODE>(s.z, factor),
                fold_finish<MODE>(s.w, factor)};
      *reinterpret_cast<f32x4*>(out + gidx * 4) = s;
    }
    done = groups * 4;
  }
  for (int64_t i = done + tid; i < n; i += nthreads) {
    float s = fold_term<MODE>(src[i], factor);
    for (int r = 1; r < world; ++r) s = s + fold_term<MODE>(src[r * stride + i], factor);
    out[i] = fold_finish<MODE>(s, factor);
  }
}

// The same fold over bf16 contributions: every term is widened to fp32 (and
// pre-multiplied if asked), the terms are added in fp32 in rank order, and the
// result is rounded to bf16 once.
template <int MODE>
__global__ __launch_bounds__(kThreads) void reduce_rows_bf16_kernel(uint16_t* __restrict__ out,
                                                                   const uint16_t* __restrict__ src,
                                                                   int64_t stride, int world, int64_t n,
                                                                   float factor, int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gidx = tid; gidx < groups; gidx += nthreads) {
      float s[8], v[8];
      unpack8(load_stream_u32x4(src + gidx * 8), s);
#pragma unroll
      for (int j = 0; j < 8; ++j) s[j] = fold_term<MODE>(s[j], factor);
      for (int r = 1; r < world; ++r) {
        unpack8(load_stream_u32x4(src + r * stride + gidx * 8), v);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[j] = s[j] + fold_term<MODE>(v[j], factor);
      }
      uint32_t bits[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) bits[j] = f32_to_bf16_bits(fold_finish<MODE>(s[j], factor));
      *reinterpret_cast<u32x4*>(out + gidx * 8) = pack8(bits);
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads) {
    float s = fold_term<MODE>(bf16_bits_to_f32(src[i]), factor);
    for (int r = 1; r < world; ++r) s = s + fold_term<MODE>(bf16_bits_to_f32(src[r * stride + i]), factor);
    out[i] = static_cast<uint16_t>(f32_to_bf16_bits(fold_finish<MODE>(s, factor)));
  }
}

// m = bf16(lerp(m, g, 1-mu)); out = nesterov ? bf16(lerp(g, m, mu)) : m.
// 8 elements (16 bytes) per thread and iteration when the three pointers are
// 16-byte aligned, then a scalar tail; scalar throughout otherwise.
__global__ __launch_bounds__(kThreads) void muon_prepare_kernel(uint16_t* __restrict__ mom,
                                                               const uint16_t* __restrict__ grad,
                                                               uint16_t* __restrict__ out, int64_t n,
                                                               float one_minus_mu, float mu, int nesterov,
                                                               int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gi = tid; gi < groups; gi += nthreads) {
      float m[8], g[8];
      unpack8(load_stream_u32x4(mom + gi * 8), m);
      unpack8(load_stream_u32x4(grad + gi * 8), g);
      uint32_t mb[8], ob[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) muon_prepare_one(m[j], g[j], one_minus_mu, mu, nesterov, &mb[j], &ob[j]);
      store_stream_u32x4(mom + gi * 8, pack8(mb));
      store_stream_u32x4(out + gi * 8, pack8(ob));
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads) {
    uint32_t mb, ob;
    muon_prepare_one(bf16_bits_to_f32(mom[i]), bf16_bits_to_f32(grad[i]), one_minus_mu, mu, nesterov, &mb, &ob);
    mom[i] = static_cast<uint16_t>(mb);
    out[i] = static_cast<uint16_t>(ob);
  }
}

// p = bf16(p * decay); p = bf16(p + neg_lr * d'), d' = scale == 1 ? d : bf16(d * scale).
__global__ __launch_bounds__(kThreads) void muon_apply_kernel(uint16_t* __restrict__ param,
                                                             const uint16_t* __restrict__ dir, int64_t n,
                                                             float decay, float neg_lr, float dir_scale,
                                                             int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gi = tid; gi < groups; gi += nthreads) {
      float pv[8], dv[8];
      unpack8(load_stream_u32x4(param + gi * 8), pv);
      unpack8(load_stream_u32x4(dir + gi * 8), dv);
      uint32_t pb[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) pb[j] = muon_apply_one(pv[j], dv[j], decay, neg_lr, dir_scale);
      store_stream_u32x4(param + gi * 8, pack8(pb));
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads)
    param[i] = static_cast<uint16_t>(
        muon_apply_one(bf16_bits_to_f32(param[i]), bf16_bits_to_f32(dir[i]), decay, neg_lr, dir_scale));
}

// fp32 master state: m = lerp(m, g, 1-mu) stays fp32; out = bf16 of the
// Nesterov blend (or of m), the input of the orthogonalization.
__global__ __launch_bounds__(kThreads) void muon_prepare_f32_kernel(float* __restrict__ mom,
                                                                   const float* __restrict__ grad,
                                                                   uint16_t* __restrict__ out, int64_t n,
                                                                   float one_minus_mu, float mu, int nesterov,
                                                                   int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gi = tid; gi < groups; gi += nthreads) {
      float m[8], g[8];
      load8_f32(mom + gi * 8, m);
      load8_f32(grad + gi * 8, g);
      uint32_t ob[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) muon_prepare_one_f32(m[j], g[j], one_minus_mu, mu, nesterov, &m[j], &ob[j]);
      store8_f32(mom + gi * 8, m);
      store_stream_u32x4(out + gi * 8, pack8(ob));
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads) {
    float m;
    uint32_t ob;
    muon_prepare_one_f32(mom[i], grad[i], one_minus_mu, mu, nesterov, &m, &ob);
    mom[i] = m;
    out[i] = static_cast<uint16_t>(ob);
  }
}

// p = p * decay; p = p + neg_lr * d', d' = scale == 1 ? d : d * scale, all fp32; d is bf16.
__global__ __launch_bounds__(kThreads) void muon_apply_f32_kernel(float* __restrict__ param,
                                                                 const uint16_t* __restrict__ dir, int64_t n,
                                                                 float decay, float neg_lr, float dir_scale,
                                                                 int vec_ok) {
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t nthreads = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t groups = n / 8;
    for (int64_t gi = tid; gi < groups; gi += nthreads) {
      float pv[8], dv[8];
      load8_f32(param + gi * 8, pv);
      unpack8(load_stream_u32x4(dir + gi * 8), dv);
#pragma unroll
      for (int j = 0; j < 8; ++j) pv[j] = muon_apply_one_f32(pv[j], dv[j], decay, neg_lr, dir_scale);
      store8_f32(param + gi * 8, pv);
    }
    done = groups * 8;
  }
  for (int64_t i = done + tid; i < n; i += nthreads)
    param[i] = muon_apply_one_f32(param[i], bf16_bits_to_f32(dir[i]), decay, neg_lr, dir_scale);
}

}  // namespace
}  // namespace fsh

FSH_API int fsh_accumulate_grad(float* acc_dev, const void* grad_dev, int32_t grad_dtype, int64_t numel,
                                int32_t overwrite, void* stream) {
  using namespace fsh;
  if (numel < 0) return fail(FSH_EINVAL, "fsh_accumulate_grad: negative numel");
  if (numel == 0) return FSH_OK;
  if (!acc_dev || !grad_dev) return fail(FSH_EINVAL, "fsh_accumulate_grad: null pointer");
  if (grad_dtype != FSH_DT_BF16 && grad_dtype != FSH_DT_F32)
    return fail(FSH_EINVAL, "fsh_accumulate_grad: unsupported grad dtype %d", grad_dtype);
  if (!aligned(acc_dev, 4) || !aligned(grad_dev, grad_dtype == FSH_DT_BF16 ? 2 : 4))
    return fail(FSH_EINVAL, "fsh_accumulate_grad: pointers misaligned for their dtypes");
  const int vec_ok = aligned(acc_dev, 16) && aligned(grad_dev, 16);
  const dim3 g(grid_for(ceil_div(numel, 8))), b(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t* grad = static_cast<const uint8_t*>(grad_dev);
  if (grad_dtype == FSH_DT_BF16) {
    if (overwrite)
      hipLaunchKernelGGL((accumulate_kernel<FSH_DT_BF16, true>), g, b, 0, s, acc_dev, grad, numel, vec_ok);
    else
      hipLaunchKernelGGL((accumulate_kernel<FSH_DT_BF16, false>), g, b, 0, s, acc_dev, grad, numel, vec_ok);
  } else {
    if (overwrite)
      hipLaunchKernelGGL((accumulate_kernel<FSH_DT_F32, true>), g, b, 0, s, acc_dev, grad, numel, vec_ok);
    else
      hipLaunchKernelGGL((accumulate_kernel<FSH_DT_F32, false>), g, b, 0, s, acc_dev, grad, numel, vec_ok);
  }
  return check_launch("fsh_accumulate_grad");
}

FSH_API int fsh_reduce_rows_f32(float* out_dev, const float* src_dev, int64_t contribution_stride,
                                int32_t world, int64_t column_offset, int64_t numel, int32_t mode,
                                float factor, void* stream) {
  using namespace fsh;
  if (numel < 0 || world <= 0 || column_offset < 0 || contribution_stride < 0)
    return fail(FSH_EINVAL, "fsh_reduce_rows_f32: bad sizes (world %d, numel %lld)", world, (long long)numel);
  if (numel == 0) return FSH_OK;
  if (!out_dev || !src_dev) return fail(FSH_EINVAL, "fsh_reduce_rows_f32: null pointer");
  if (!aligned(out_dev, 4) || !aligned(src_dev, 4)) return fail(FSH_EINVAL, "fsh_reduce_rows_f32: misaligned");
  if (mode < FSH_REDUCE_SUM || mode > FSH_REDUCE_POSTDIV)
    return fail(FSH_EINVAL, "fsh_reduce_rows_f32: unknown mode %d", mode);
  const float* src = src_dev + column_offset;
  const int vec_ok = aligned(out_dev, 16) && aligned(src, 16) && (contribution_stride % 4 == 0);
  const dim3 g(grid_for(ceil_div(numel, 4))), b(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (mode) {
    case FSH_REDUCE_SUM:
      hipLaunchKernelGGL((reduce_rows_kernel<FSH_REDUCE_SUM>), g, b, 0, s, out_dev, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    case FSH_REDUCE_PREMUL:
      hipLaunchKernelGGL((reduce_rows_kernel<FSH_REDUCE_PREMUL>), g, b, 0, s, out_dev, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    case FSH_REDUCE_POSTMUL:
      hipLaunchKernelGGL((reduce_rows_kernel<FSH_REDUCE_POSTMUL>), g, b, 0, s, out_dev, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    default:
      hipLaunchKernelGGL((reduce_rows_kernel<FSH_REDUCE_POSTDIV>), g, b, 0, s, out_dev, src, contribution_stride, world, numel, factor, vec_ok);
      break;
  }
  return check_launch("fsh_reduce_rows_f32");
}

FSH_API int fsh_muon_prepare(void* momentum_dev, const void* grad_dev, void* out_dev, int64_t numel,
                             float lerp_weight, float nesterov_weight, int32_t nesterov, void* stream) {
  using namespace fsh;
  if (numel < 0) return fail(FSH_EINVAL, "fsh_muon_prepare: negative numel");
  if (numel == 0) return FSH_OK;
  if (!momentum_dev || !grad_dev || !out_dev) return fail(FSH_EINVAL, "fsh_muon_prepare: null pointer");
  if (!aligned(momentum_dev, 2) || !aligned(grad_dev, 2) || !aligned(out_dev, 2))
    return fail(FSH_EINVAL, "fsh_muon_prepare: pointers misaligned for bf16");
  const int vec_ok = aligned(momentum_dev, 16) && aligned(grad_dev, 16) && aligned(out_dev, 16);
  hipLaunchKernelGGL(muon_prepare_kernel, dim3(grid_for(ceil_div(numel, 8))), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint16_t*>(momentum_dev),
                     static_cast<const uint16_t*>(grad_dev), static_cast<uint16_t*>(out_dev), numel,
                     lerp_weight, nesterov_weight, nesterov, vec_ok);
  return check_launch("fsh_muon_prepare");
}

FSH_API int fsh_muon_apply(void* param_dev, const void* direction_dev, int64_t numel, float decay_factor,
                           float neg_adjusted_lr, float direction_scale, void* stream) {
  using namespace fsh;
  if (numel < 0) return fail(FSH_EINVAL, "fsh_muon_apply: negative numel");
  if (numel == 0) return FSH_OK;
  if (!param_dev || !direction_dev) return fail(FSH_EINVAL, "fsh_muon_apply: null pointer");
  if (!aligned(param_dev, 2) || !aligned(direction_dev, 2))
    return fail(FSH_EINVAL, "fsh_muon_apply: pointers misaligned for bf16");
  const int vec_ok = aligned(param_dev, 16) && aligned(direction_dev, 16);
  hipLaunchKernelGGL(muon_apply_kernel, dim3(grid_for(ceil_div(numel, 8))), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint16_t*>(param_dev),
                     static_cast<const uint16_t*>(direction_dev), numel, decay_factor, neg_adjusted_lr,
                     direction_scale, vec_ok);
  return check_launch("fsh_muon_apply");
}

FSH_API int fsh_muon_prepare_f32(float* momentum_dev, const float* grad_dev, void* out_dev, int64_t numel,
                                 float lerp_weight, float nesterov_weight, int32_t nesterov, void* stream) {
  using namespace fsh;
  if (numel < 0) return fail(FSH_EINVAL, "fsh_muon_prepare_f32: negative numel");
  if (numel == 0) return FSH_OK;
  if (!momentum_dev || !grad_dev || !out_dev) return fail(FSH_EINVAL, "fsh_muon_prepare_f32: null pointer");
  if (!aligned(momentum_dev, 4) || !aligned(grad_dev, 4) || !aligned(out_dev, 2))
    return fail(FSH_EINVAL, "fsh_muon_prepare_f32: pointers misaligned for their dtypes");
  const int vec_ok = aligned(momentum_dev, 16) && aligned(grad_dev, 16) && aligned(out_dev, 16);
  hipLaunchKernelGGL(muon_prepare_f32_kernel, dim3(grid_for(ceil_div(numel, 8))), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), momentum_dev, grad_dev, static_cast<uint16_t*>(out_dev), numel,
                     lerp_weight, nesterov_weight, nesterov, vec_ok);
  return check_launch("fsh_muon_prepare_f32");
}

FSH_API int fsh_muon_apply_f32(float* param_dev, const void* direction_dev, int64_t numel, float decay_factor,
                               float neg_adjusted_lr, float direction_scale, void* stream) {
  using namespace fsh;
  if (numel < 0) return fail(FSH_EINVAL, "fsh_muon_apply_f32: negative numel");
  if (numel == 0) return FSH_OK;
  if (!param_dev || !direction_dev) return fail(FSH_EINVAL, "fsh_muon_apply_f32: null pointer");
  if (!aligned(param_dev, 4) || !aligned(direction_dev, 2))
    return fail(FSH_EINVAL, "fsh_muon_apply_f32: pointers misaligned for their dtypes");
  const int vec_ok = aligned(param_dev, 16) && aligned(direction_dev, 16);
  hipLaunchKernelGGL(muon_apply_f32_kernel, dim3(grid_for(ceil_div(numel, 8))), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), param_dev, static_cast<const uint16_t*>(direction_dev), numel,
                     decay_factor, neg_adjusted_lr, direction_scale, vec_ok);
  return check_launch("fsh_muon_apply_f32");
}

FSH_API int fsh_reduce_rows_bf16(void* out_dev, const void* src_dev, int64_t contribution_stride, int32_t world,
                                 int64_t column_offset, int64_t numel, int32_t mode, float factor, void* stream) {
  using namespace fsh;
  if (numel < 0 || world <= 0 || column_offset < 0 || contribution_stride < 0)
    return fail(FSH_EINVAL, "fsh_reduce_rows_bf16: bad sizes (world %d, numel %lld)", world, (long long)numel);
  if (numel == 0) return FSH_OK;
  if (!out_dev || !src_dev) return fail(FSH_EINVAL, "fsh_reduce_rows_bf16: null pointer");
  if (!aligned(out_dev, 2) || !aligned(src_dev, 2)) return fail(FSH_EINVAL, "fsh_reduce_rows_bf16: misaligned");
  if (mode < FSH_REDUCE_SUM || mode > FSH_REDUCE_POSTDIV)
    return fail(FSH_EINVAL, "fsh_reduce_rows_bf16: unknown mode %d", mode);
  const uint16_t* src = static_cast<const uint16_t*>(src_dev) + column_offset;
  uint16_t* out = static_cast<uint16_t*>(out_dev);
  const int vec_ok = aligned(out, 16) && aligned(src, 16) && (contribution_stride % 8 == 0);
  const dim3 g(grid_for(ceil_div(numel, 8))), b(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (mode) {
    case FSH_REDUCE_SUM:
      hipLaunchKernelGGL((reduce_rows_bf16_kernel<FSH_REDUCE_SUM>), g, b, 0, s, out, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    case FSH_REDUCE_PREMUL:
      hipLaunchKernelGGL((reduce_rows_bf16_kernel<FSH_REDUCE_PREMUL>), g, b, 0, s, out, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    case FSH_REDUCE_POSTMUL:
      hipLaunchKernelGGL((reduce_rows_bf16_kernel<FSH_REDUCE_POSTMUL>), g, b, 0, s, out, src, contribution_stride, world, numel, factor, vec_ok);
      break;
    default:
      hipLaunchKernelGGL((reduce_rows_bf16_kernel<FSH_REDUCE_POSTDIV>), g, b, 0, s, out, src, contribution_stride, world, numel, factor, vec_ok);
      break;
  }
  return check_launch("fsh_reduce_rows_bf16");
}
