// The arithmetic of a head's RMSNorm and rotation, element by element, shared by the
// kernel that normalises, rotates and stores q|k|v (rope_kv.hip) and by the decode
// attention that does the same for its own token in its prologue (attention.hip): the
// same expressions compiled from the same source, so both give the same bits.
// (/root/reference/src/transformer/hybrid_attn.zig:371-382 for the norm before the
// rotation, /root/reference/src/cuda/layer_kernels.cu:353-365 for the pairing (p, p + half).)
#pragma once
#include "common.h"

// sum of squares of eight consecutive elements, in their order
__device__ __forceinline__ float rope_sum_squares8(const float (&x)[8]) {
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
  return ss;
}

__device__ __forceinline__ float rope_rms_scale(float sum_squares, int d, float eps) {
  return 1.0f / sqrtf(sum_squares / (float)d + eps);
}

__device__ __forceinline__ void rope_scale8(float (&x)[8], float scale, const float (&w)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = x[i] * scale * w[i];
}

// element p of the lower half with its partner p + half, and the partner's own result
__device__ __forceinline__ float rope_rotate_low(float x, float other, float cs, float sn) {
  return x * cs - other * sn;
}
__device__ __forceinline__ float rope_rotate_high(float x, float other, float cs, float sn) {
  return other * sn + x * cs;
}

// cosine and sine of position * inv_freq[p]
__device__ __forceinline__ void rope_angle(int position, float inv_freq, float* cs, float* sn) {
  const float angle = (float)position * inv_freq;
  sincosf(angle, sn, cs);
}
