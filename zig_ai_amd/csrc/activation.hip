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

// Columns [col0, col0 + ncols) of every row of `in` [rows, in_width] into columns
// [out_col0, out_col0 + ncols) of `out` [rows, out_width], converted between the two
// storage types: how a mixer takes q, k and v out of a fused projection's rows and puts
// them back side by side, without the tensor library.
template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
copy_columns_kernel(const TI* __restrict__ in, TO* __restrict__ out, int in_width, int col0,
                    int out_width, int out_col0, int ncols, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / ncols;
  const int c = (int)(idx % ncols);
  out[row * out_width + out_col0 + c] = from_f32<TO>(to_f32<TI>(in[row * in_width + col0 + c]));
}

extern "C" int za_copy_columns(const void* in, int in_dtype, int in_width, int col0, void* out,
                               int out_dtype, int out_width, int out_col0, int rows, int ncols,
                               hipStream_t stream) {
  if (rows == 0 || ncols == 0) return 0;
  if (rows < 0 || ncols < 0 || !in || !out || col0 < 0 || out_col0 < 0 ||
      col0 + ncols > in_width || out_col0 + ncols > out_width)
    return ZA_ERR_ARG;
  const size_t total = (size_t)rows * ncols;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
#define ZA_COPY_COLUMNS(TI, TO)                                                                   \
  hipLaunchKernelGGL((copy_columns_kernel<TI, TO>), grid, block, 0, stream, (const TI*)in, (TO*)out, \
                     in_width, col0, out_width, out_col0, ncols, total)
  if (in_dtype == 0 && out_dtype == 0) ZA_COPY_COLUMNS(float, float);
  else if (in_dtype == 0 && out_dtype == 1) ZA_COPY_COLUMNS(float, bf16_t);
  else if (in_dtype == 1 && out_dtype == 0) ZA_COPY_COLUMNS(bf16_t, float);
  else if (in_dtype == 1 && out_dtype == 1) ZA_COPY_COLUMNS(bf16_t, bf16_t);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_COPY_COLUMNS
  return za_launch_status();
}
