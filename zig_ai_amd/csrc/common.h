// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wavefront (64 lanes) and workgroup reductions, 16-byte vector access.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ZA_WAVE 64

typedef __bf16 bf16_t;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// Every launcher returns 0 on success or a hipError_t; bad arguments return one
// of these negative codes without launching anything.
#define ZA_ERR_ARG (-1)
#define ZA_ERR_UNSUPPORTED (-2)

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// Round to nearest even, the conversion the hardware instruction performs.
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = ZA_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, ZA_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = ZA_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, ZA_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of shared memory and may be reused after
// the call returns.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (ZA_WAVE - 1);
  const int wave = threadIdx.x / ZA_WAVE;
  const int nwaves = (blockDim.x + ZA_WAVE - 1) / ZA_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += scratch[i];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (ZA_WAVE - 1);
  const int wave = threadIdx.x / ZA_WAVE;
  const int nwaves = (blockDim.x + ZA_WAVE - 1) / ZA_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float best = scratch[0];
  for (int i = 1; i < nwaves; ++i) best = fmaxf(best, scratch[i]);
  return best;
}

// Eight consecutive elements as floats.  `p` must be 16-byte aligned for
// bfloat16 and for float.
template <typename T> __device__ __forceinline__ void load8(const T* p, float out[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float out[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
  out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
template <> __device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float out[8]) {
  const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = (float)v[i];
}

template <typename T> __device__ __forceinline__ void store8(T* p, const float in[8]);
template <> __device__ __forceinline__ void store8<float>(float* p, const float in[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(in[4], in[5], in[6], in[7]);
}
template <> __device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float in[8]) {
  bf16x8_t v;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (bf16_t)in[i];
  *reinterpret_cast<bf16x8_t*>(p) = v;
}

static inline int za_launch_status() { return (int)hipGetLastError(); }
