// RMSNorm, optionally fused with the residual add that precedes it, and the
// embedding row gather that starts the residual stream.
//
//   h   = residual (32-bit, may be absent) + delta (storage type, may be absent)
//   out = h * (1 / sqrt(mean(h^2) + eps)) * weight
//
// The residual stream stays in 32-bit; with `write_residual` the sum is stored
// back so that the next block adds to it.  With `rows` only the listed rows are
// normalised (the rows whose logits are wanted) and nothing is stored back.
// Formula as in /root/reference/src/transformer/norm.zig:6-33 (32-bit sum of
// squares, weight multiplied after the scale, no bias).
#include "common.h"

template <typename TD, typename TO>
__global__ void __launch_bounds__(256)
add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                   const float* __restrict__ weight, TO* __restrict__ out,
                   const int* __restrict__ rows, int width, float eps, int write_residual) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* x = residual ? residual + src * width : nullptr;
  const TD* dl = delta ? delta + src * width : nullptr;
  TO* o = out + (size_t)r * width;

  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float h = x ? x[i] : 0.f;
    if (dl) h += to_f32<TD>(dl[i]);
    if (write_residual) x[i] = h;
    ss += h * h;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float h;
    if (write_residual) {
      h = x[i];  // this thread stored it above
    } else {
      h = x ? x[i] : 0.f;
      if (dl) h += to_f32<TD>(dl[i]);
    }
    o[i] = from_f32<TO>(h * scale * weight[i]);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
embed_gather_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                    float* __restrict__ out, int width, int vocab) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  float* o = out + (size_t)t * width;
  if (tok < 0 || tok >= vocab) {
    // Never read outside the table; an id the host failed to reject poisons its row.
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = __builtin_nanf("");
    return;
  }
  const T* row = table + (size_t)tok * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = to_f32<T>(row[i]);
}

// dtype codes: 0 = float32, 1 = bfloat16
extern "C" int za_add_rmsnorm(void* residual, const void* delta, int delta_dtype,
                              const float* weight, void* out, int out_dtype, const int* rows,
                              int n_rows, int width, float eps, int write_residual,
                              hipStream_t stream) {
  if (n_rows == 0) return 0;
  if (n_rows < 0 || width <= 0 || (!residual && !delta) || !weight || !out) return ZA_ERR_ARG;
  if (!residual || rows) write_residual = 0;
  dim3 grid(n_rows), block(256);
  float* res = (float*)residual;
#define ZA_NORM_CASE(DD, TD, OD, TO)                                                        \
  if (delta_dtype == DD && out_dtype == OD) {                                               \
    hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TO>), grid, block, 0, stream, res,           \
                       (const TD*)delta, weight, (TO*)out, rows, width, eps, write_residual); \
    return za_launch_status();                                                              \
  }
  ZA_NORM_CASE(0, float, 0, float)
  ZA_NORM_CASE(0, float, 1, bf16_t)
  ZA_NORM_CASE(1, bf16_t, 0, float)
  ZA_NORM_CASE(1, bf16_t, 1, bf16_t)
#undef ZA_NORM_CASE
  return ZA_ERR_UNSUPPORTED;
}

extern "C" int za_embed_gather(const int* tokens, const void* table, int table_dtype, float* out,
                               int n_tokens, int width, int vocab, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || width <= 0 || vocab <= 0 || !tokens || !table || !out) return ZA_ERR_ARG;
  dim3 grid(n_tokens), block(256);
  if (table_dtype == 0) {
    hipLaunchKernelGGL((embed_gather_kernel<float>), grid, block, 0, stream, tokens,
                       (const float*)table, out, width, vocab);
  } else if (table_dtype == 1) {
    hipLaunchKernelGGL((embed_gather_kernel<bf16_t>), grid, block, 0, stream, tokens,
                       (const bf16_t*)table, out, width, vocab);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
  return za_launch_status();
}
