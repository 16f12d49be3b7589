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

}  // namespace fsh
