// The ShortConv mixer between its two projections: input gate, causal
// depth-wise convolution over the request's own past, output gate, and the
// update of the request's carried state.
//
//   z = in_proj(x) = [B | C | X] per token (three blocks of `width` channels)
//   u[t]   = B[t] * X[t]
//   c[t]   = bias + sum_{j<L} w[ch][j] * u[t - (L-1) + j]      (u before the portion comes
//                                                               from the request's state)
//   y[t]   = C[t] * c[t]
//   state <- the last L values of u, oldest first  (state[slot] starts slot_stride floats
//            after state[slot - 1]; within a slot the layout is [channel][L])
//
// The reference's kernel has the same mechanics (taps over [state rows; new rows],
// then the state becomes the last rows: /root/reference/src/cuda/layer_kernels.cu:192-222,
// /root/reference/src/transformer/short_conv.zig:188-225) around a different
// gating; the gating here is the B*x ... *C form of the model's definition.
//
// One thread per (token, channel).  Tokens are packed request after request;
// `token_seq` names each token's request, so a thread never reads across a
// request's edge.  The first token of each portion also computes the portion's
// next L-2 outputs (the only ones that need the old state) and writes the new
// state, so within a launch exactly one thread touches a given state element.
#include "common.h"

#define SC_MAX_L 8

template <typename T>
__global__ void __launch_bounds__(256)
short_conv_kernel(const T* __restrict__ z, const float* __restrict__ w,
                  const float* __restrict__ bias, float* __restrict__ state,
                  const int* __restrict__ token_seq, const int* __restrict__ seq_start,
                  const int* __restrict__ slot_id, T* __restrict__ y, int width, int L,
                  long long slot_stride) {
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (ch >= width) return;
  const int s = token_seq[t];
  const int first = seq_start[s];
  const int n = seq_start[s + 1] - first;
  const int qi = t - first;
  if (qi > 0 && qi < L - 1) return;  // served by the portion's first token

  float wt[SC_MAX_L];
#pragma unroll
  for (int j = 0; j < SC_MAX_L; ++j) wt[j] = j < L ? w[(size_t)ch * L + j] : 0.f;
  const float b = bias ? bias[ch] : 0.f;
  const size_t zs = (size_t)3 * width;  // row stride of z

  auto gate_in = [&](int row) -> float {
    const T* zr = z + (size_t)row * zs;
    return to_f32<T>(zr[ch]) * to_f32<T>(zr[2 * width + ch]);
  };
  auto gate_out = [&](int row, float c) -> T {
    return from_f32<T>(to_f32<T>(z[(size_t)row * zs + width + ch]) * c);
  };

  if (qi > 0) {  // qi >= L - 1: every input it needs lies in this portion
    float c = b;
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j < L) c = fmaf(wt[j], gate_in(t - (L - 1) + j), c);
    y[(size_t)t * width + ch] = gate_out(t, c);
    return;
  }

  // qi == 0: the outputs that reach into the carried state, then the new state.
  float* st = state + (size_t)slot_id[s] * (size_t)slot_stride + (size_t)ch * L;
  float hist[SC_MAX_L];  // hist[0..L-1]: the last L inputs, oldest first
#pragma unroll
  for (int j = 0; j < SC_MAX_L; ++j) hist[j] = j < L ? st[j] : 0.f;
  const int reach = L > 1 ? L - 1 : 1;  // tokens this thread serves
  const int head = n < reach ? n : reach;
  for (int i = 0; i < head; ++i) {
    const float u = gate_in(t + i);
#pragma unroll
    for (int j = 0; j < SC_MAX_L - 1; ++j)
      if (j < L - 1) hist[j] = hist[j + 1];
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j == L - 1) hist[j] = u;
    float c = b;
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j < L) c = fmaf(wt[j], hist[j], c);
    y[(size_t)(t + i) * width + ch] = gate_out(t + i, c);
  }
  if (n >= L) {
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j < L) st[j] = gate_in(first + n - L + j);
  } else {
    // n < L: every new input was shifted into hist above
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j < L) st[j] = hist[j];
  }
}

extern "C" int za_short_conv(const void* z, const float* w, const float* bias, float* state,
                             const int* token_seq, const int* seq_start, const int* slot_id,
                             void* y, int dtype, int n_tokens, int width, int L,
                             long long slot_stride, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || width <= 0 || L <= 0 || !z || !w || !state || !token_seq || !seq_start ||
      !slot_id || !y || slot_stride < (long long)width * L)
    return ZA_ERR_ARG;
  if (L > SC_MAX_L || (width + 255) / 256 > 65535) return ZA_ERR_UNSUPPORTED;
  dim3 grid(n_tokens, (width + 255) / 256), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL((short_conv_kernel<float>), grid, block, 0, stream, (const float*)z, w,
                       bias, state, token_seq, seq_start, slot_id, (float*)y, width, L, slot_stride);
  else if (dtype == 1)
    hipLaunchKernelGGL((short_conv_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)z, w,
                       bias, state, token_seq, seq_start, slot_id, (bf16_t*)y, width, L, slot_stride);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}
