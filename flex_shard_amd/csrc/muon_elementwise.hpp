// Per-element arithmetic of the Muon momentum and update steps, shared by
// the per-tensor kernels and the batched whole-step kernels: fp32 math with
// one bf16 rounding per tensor op of the reference
// (dist_muon/optimizer.py:2049-2068, :2100-2117).
#pragma once
#include "common.hpp"

namespace fsh {

// torch.lerp(start, end, w) in fp32: w < 0.5 ? start + w*(end-start)
//                                            : end - (end-start)*(1-w).
__device__ __forceinline__ float lerp_f32(float start, float end, float w) {
  const float diff = end - start;
  return w < 0.5f ? start + w * diff : end - diff * (1.0f - w);
}

// Eight bf16 values of a 16-byte vector as floats, and back.
__device__ __forceinline__ void unpack8(const u32x4 v, float* f) {
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = u32_as_f32(d[j] << 16);
    f[2 * j + 1] = u32_as_f32(d[j] & 0xFFFF0000u);
  }
}
__device__ __forceinline__ u32x4 pack8(const uint32_t* bits) {
  return u32x4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16), bits[4] | (bits[5] << 16),
               bits[6] | (bits[7] << 16)};
}

__device__ __forceinline__ void muon_prepare_one(float m, float g, float one_minus_mu, float mu, int nesterov,
                                                 uint32_t* m_bits, uint32_t* out_bits) {
  *m_bits = f32_to_bf16_bits(lerp_f32(m, g, one_minus_mu));
  *out_bits = nesterov ? f32_to_bf16_bits(lerp_f32(g, bf16_bits_to_f32(*m_bits), mu)) : *m_bits;
}

__device__ __forceinline__ uint32_t muon_apply_one(float p, float d, float decay, float neg_lr, float dir_scale) {
  if (dir_scale != 1.0f) d = bf16_bits_to_f32(f32_to_bf16_bits(d * dir_scale));
  p = bf16_bits_to_f32(f32_to_bf16_bits(p * decay));
  return f32_to_bf16_bits(p + neg_lr * d);
}

// The same two steps on fp32 master state (fp32 gradient, momentum buffer and
// parameter): nothing is rounded to bf16 except the Newton-Schulz input, which
// the orthogonalization casts (dist_muon/optimizer.py:2131), and the scaled
// direction stays in fp32 as it does in the reference's fp32 buffer.
__device__ __forceinline__ void muon_prepare_one_f32(float m, float g, float one_minus_mu, float mu, int nesterov,
                                                     float* m_out, uint32_t* out_bits) {
  *m_out = lerp_f32(m, g, one_minus_mu);
  *out_bits = f32_to_bf16_bits(nesterov ? lerp_f32(g, *m_out, mu) : *m_out);
}

__device__ __forceinline__ float muon_apply_one_f32(float p, float d, float decay, float neg_lr, float dir_scale) {
  if (dir_scale != 1.0f) d = d * dir_scale;
  p = p * decay;
  return p + neg_lr * d;
}

// Eight fp32 values at a 16-byte aligned address, and back.
__device__ __forceinline__ void load8_f32(const float* src, float* f) {
  const f32x4 a = load_stream_f32x4(src), b = load_stream_f32x4(src + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
  f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void store8_f32(float* dst, const float* f) {
  *reinterpret_cast<f32x4*>(dst) = f32x4{f[0], f[1], f[2], f[3]};
  *reinterpret_cast<f32x4*>(dst + 4) = f32x4{f[4], f[5], f[6], f[7]};
}

}  // namespace fsh
