// What this GPU does at best, for the benchmark's fractions: a stream of reads from
// memory, and matrix-core instructions issued back to back from registers.  Neither is
// part of a step; they give the measured ceilings that the published peaks are held
// against (the reference quotes no ceilings at all: it reports tokens per second,
// /root/reference/src/main.zig:1409-1432).
#include "common.h"

// Every thread reads 16-byte pieces a whole grid apart and keeps a sum that is stored
// once (so that the reads cannot be dropped).
__global__ void __launch_bounds__(256)
read_stream_kernel(const f32x4_t* __restrict__ src, size_t n_vec, float* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const f32x4_t a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc += a + b + c + d;
  }
  for (; i < n_vec; i += stride) acc += src[i];
  const float s = acc[0] + acc[1] + acc[2] + acc[3];
  if (s == 123456.789f) sink[0] = s;      // (never true for the zeros and ones it is run on)
}

// `iters` rounds of eight independent 16x16x32 bfloat16 products per wave, operands and
// accumulators in registers: 8 * 2 * 16 * 16 * 32 flop per wave and round.
__global__ void __launch_bounds__(256)
mfma_loop_kernel(int iters, float* __restrict__ sink) {
  bf16x8_t a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16_t)(float)((threadIdx.x + i) & 3);
    b[i] = (bf16_t)(float)((threadIdx.x * 3 + i) & 1);
  }
  f32x4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  if (s == -1.0f) sink[0] = s;            // (sums of non-negative products: never true)
}

// Reads `bytes` (a multiple of 16) from `src` once, with `blocks` workgroups.
extern "C" int za_read_stream(const void* src, size_t bytes, int blocks, float* sink,
                              hipStream_t stream) {
  if (!src || !sink || blocks <= 0 || bytes % 16 != 0) return ZA_ERR_ARG;
  hipLaunchKernelGGL(read_stream_kernel, dim3(blocks), dim3(256), 0, stream,
                     (const f32x4_t*)src, bytes / 16, sink);
  return za_launch_status();
}

// `blocks` workgroups of four waves, `iters` rounds each; the flop count is
// blocks * 4 * iters * 8 * 16384.
extern "C" int za_mfma_loop(int blocks, int iters, float* sink, hipStream_t stream) {
  if (!sink || blocks <= 0 || iters <= 0) return ZA_ERR_ARG;
  hipLaunchKernelGGL(mfma_loop_kernel, dim3(blocks), dim3(256), 0, stream, iters, sink);
  return za_launch_status();
}
