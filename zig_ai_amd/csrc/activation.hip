// SwiGLU gate on the fused gate|up projection:
//   out[t, i] = silu(gu[t, i]) * gu[t, I + i],   silu(g) = g / (1 + exp(-g))
// computed in 32-bit (/root/reference/src/transformer/ffn.zig:24-30,
// /root/reference/src/cuda/layer_kernels.cu:62-70).
// Also the element-wise cast between storage types.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  const float g = to_f32<T>(gu[t * 2 * inter + i]);
  const float u = to_f32<T>(gu[t * 2 * inter + inter + i]);
  const float sig = 1.0f / (1.0f + expf(-g));
  out[idx] = from_f32<T>(g * sig * u);
}

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_vec8_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  float g[8], u[8], o[8];
  load8<T>(gu + t * 2 * inter + i, g);
  load8<T>(gu + t * 2 * inter + inter + i, u);
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = g[k] * (1.0f / (1.0f + expf(-g[k]))) * u[k];
  store8<T>(out + idx, o);
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n) out[idx] = from_f32<TO>(to_f32<TI>(in[idx]));
}

extern "C" int za_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter,
                         hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || inter <= 0 || !gu || !out) return ZA_ERR_ARG;
  const size_t total = (size_t)n_tokens * inter;
  const bool vec = inter % 8 == 0;
  const size_t threads = vec ? total / 8 : total;
  dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  if (dtype == 0) {
    if (vec)
      hipLaunchKernelGGL((swiglu_vec8_kernel<float>), grid, block, 0, stream, (const float*)gu,
                         (float*)out, n_tokens, inter);
    else
      hipLaunchKernelGGL((swiglu_kernel<float>), grid, block, 0, stream, (const float*)gu,
                         (float*)out, n_tokens, inter);
  } else if (dtype == 1) {
    if (vec)
      hipLaunchKernelGGL((swiglu_vec8_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)gu,
                         (bf16_t*)out, n_tokens, inter);
    else
      hipLaunchKernelGGL((swiglu_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)gu,
                         (bf16_t*)out, n_tokens, inter);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
  return za_launch_status();
}

// dtype codes: 0 = float32, 1 = bfloat16
extern "C" int za_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                       hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || !in || !out) return ZA_ERR_ARG;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (in_dtype == 0 && out_dtype == 1)
    hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)in,
                       (bf16_t*)out, (size_t)n);
  else if (in_dtype == 1 && out_dtype == 0)
    hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)in,
                       (float*)out, (size_t)n);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}
