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

// `delta` may be a stack of `n_partials` partial sums (each `partial_stride`
// elements apart): the pieces a projection split along K leaves to its consumer.
// They are added up first, in their order, and the sum is added to the residual.
template <typename TD>
__device__ __forceinline__ float delta_at(const TD* dl, size_t i, int n_partials,
                                          size_t partial_stride) {
  float v = to_f32<TD>(dl[i]);
  for (int p = 1; p < n_partials; ++p) v += to_f32<TD>(dl[i + p * partial_stride]);
  return v;
}

// Four consecutive elements as floats; `p` aligned to four elements.
template <typename T> __device__ __forceinline__ void load4(const T* p, float out[4]);
template <> __device__ __forceinline__ void load4<float>(const float* p, float out[4]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float out[4]) {
  const bf16x4_t v = *reinterpret_cast<const bf16x4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = (float)v[i];
}
template <typename T> __device__ __forceinline__ void store4(T* p, const float in[4]);
template <> __device__ __forceinline__ void store4<float>(float* p, const float in[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float in[4]) {
  bf16x4_t v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = (bf16_t)in[i];
  *reinterpret_cast<bf16x4_t*>(p) = v;
}

// The same sum as delta_at for the four elements at `i`, with the loads of up to
// eight partial sums issued before the first is waited for.
template <typename TD>
__device__ __forceinline__ void delta4_at(const TD* dl, size_t i, int n_partials,
                                          size_t partial_stride, float v[4]) {
  load4<TD>(dl + i, v);
  for (int p0 = 1; p0 < n_partials; p0 += 8) {
    float t[8][4];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (p0 + q < n_partials) {
        load4<TD>(dl + i + (size_t)(p0 + q) * partial_stride, t[q]);
      } else {
        t[q][0] = t[q][1] = t[q][2] = t[q][3] = 0.f;
      }
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (p0 + q < n_partials) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += t[q][e];
      }
    }
  }
}

// General form: two passes over the row, any width.
template <typename TD, typename TO>
__global__ void __launch_bounds__(256)
add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                   const float* __restrict__ weight, TO* __restrict__ out,
                   const int* __restrict__ rows, int width, float eps, int write_residual,
                   int n_partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* x = residual ? residual + src * width : nullptr;
  const TD* dl = delta ? delta + src * width : nullptr;
  TO* o = out + (size_t)r * width;

  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float h = x ? x[i] : 0.f;
    if (dl) h += delta_at<TD>(dl, i, n_partials, partial_stride);
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
      if (dl) h += delta_at<TD>(dl, i, n_partials, partial_stride);
    }
    o[i] = from_f32<TO>(h * scale * weight[i]);
  }
}

// Rows of at most 256 * 4 * VPT elements with width % 4 == 0: the row stays in
// registers between the sum of squares and the scaling, one pass over memory.
template <typename TD, typename TO, int VPT>
__global__ void __launch_bounds__(256)
add_rmsnorm_regs_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                        const float* __restrict__ weight, TO* __restrict__ out,
                        const int* __restrict__ rows, int width, float eps, int write_residual,
                        int n_partials, size_t partial_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* x = residual ? residual + src * width : nullptr;
  const TD* dl = delta ? delta + src * width : nullptr;
  TO* o = out + (size_t)r * width;
  float h[VPT][4];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int i = (threadIdx.x + v * 256) * 4;
    if (i < width) {
      if (x) {
        const float4 t = *reinterpret_cast<const float4*>(x + i);
        h[v][0] = t.x; h[v][1] = t.y; h[v][2] = t.z; h[v][3] = t.w;
      } else {
        h[v][0] = h[v][1] = h[v][2] = h[v][3] = 0.f;
      }
      if (dl) {
        float d4[4];
        delta4_at<TD>(dl, i, n_partials, partial_stride, d4);
#pragma unroll
        for (int e = 0; e < 4; ++e) h[v][e] += d4[e];
      }
      if (write_residual)
        *reinterpret_cast<float4*>(x + i) = make_float4(h[v][0], h[v][1], h[v][2], h[v][3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += h[v][e] * h[v][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int i = (threadIdx.x + v * 256) * 4;
    if (i < width) {
      const float4 w = *reinterpret_cast<const float4*>(weight + i);
      const float y[4] = {h[v][0] * scale * w.x, h[v][1] * scale * w.y, h[v][2] * scale * w.z,
                          h[v][3] * scale * w.w};
      store4<TO>(o + i, y);
    }
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
                              int n_partials, long long partial_stride, hipStream_t stream) {
  if (n_rows == 0) return 0;
  if (n_rows < 0 || width <= 0 || (!residual && !delta) || !weight || !out || n_partials < 1)
    return ZA_ERR_ARG;
  if (n_partials > 1 && (!delta || partial_stride <= 0)) return ZA_ERR_ARG;
  if (!residual || rows) write_residual = 0;
  dim3 grid(n_rows), block(256);
  float* res = (float*)residual;
  const int vpt = width % 4 == 0 ? (width / 4 + 255) / 256 : 0;   // vectors per thread
#define ZA_NORM_LAUNCH(KERNEL, TD, TO)                                                      \
  hipLaunchKernelGGL((KERNEL), grid, block, 0, stream, res, (const TD*)delta, weight,       \
                     (TO*)out, rows, width, eps, write_residual, n_partials,                \
                     (size_t)partial_stride)
#define ZA_NORM_CASE(DD, TD, OD, TO)                                                        \
  if (delta_dtype == DD && out_dtype == OD) {                                               \
    if (vpt == 1) ZA_NORM_LAUNCH((add_rmsnorm_regs_kernel<TD, TO, 1>), TD, TO);             \
    else if (vpt == 2) ZA_NORM_LAUNCH((add_rmsnorm_regs_kernel<TD, TO, 2>), TD, TO);        \
    else if (vpt >= 3 && vpt <= 4) ZA_NORM_LAUNCH((add_rmsnorm_regs_kernel<TD, TO, 4>), TD, TO); \
    else ZA_NORM_LAUNCH((add_rmsnorm_kernel<TD, TO>), TD, TO);                              \
    return za_launch_status();                                                              \
  }
  ZA_NORM_CASE(0, float, 0, float)
  ZA_NORM_CASE(0, float, 1, bf16_t)
  ZA_NORM_CASE(1, bf16_t, 0, float)
  ZA_NORM_CASE(1, bf16_t, 1, bf16_t)
#undef ZA_NORM_CASE
#undef ZA_NORM_LAUNCH
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
