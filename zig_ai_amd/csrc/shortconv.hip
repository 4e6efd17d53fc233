// The ShortConv mixer between its two projections: input gate, causal
// depth-wise convolution over the request's own past, output gate, and the
// update of the request's carried state.
//
//   z = in_proj(x) = [B | C | X] per token (three blocks of `width` channels)
//   u[t]   = B[t] * X[t]
//   c[t]   = bias + sum_{j<L} w[j][ch] * u[t - (L-1) + j]      (u before the portion comes
//                                                               from the request's state)
//   y[t]   = C[t] * c[t]
//   (the filter is given tap by tap, w[j] holding tap j of every channel: a thread's
//   channels, and neighbouring threads', then lie side by side)
//   state <- the last L values of u, oldest first  (state[slot] starts slot_stride floats
//            after state[slot - 1]; within a slot the layout is [channel][L])
//
// The reference's kernel has the same mechanics (taps over [state rows; new rows],
// then the state becomes the last rows: /root/reference/src/cuda/layer_kernels.cu:192-222,
// /root/reference/src/transformer/short_conv.zig:188-225) around a different
// gating; the gating here is the B*x ... *C form of the model's definition.
//
// Tokens are packed request after request; `token_seq` names each token's request, so
// a thread never uses inputs from across a request's edge.  Two kinds of workgroups
// share a launch (told apart by their place in the grid, heads first):
//   * body: one thread per (4 consecutive tokens, 8 channels) with 16-byte accesses
//     (one channel for widths that are no multiple of 8), for the tokens whose L
//     inputs all lie in the portion itself.  The inputs of the 4 + L - 1 rows are
//     each read once and the filter taps are kept in registers.
//   * head: one thread per (portion, channel).  It computes the portion's first L-1
//     outputs (the only ones that need the old state; one output when L = 1) and
//     writes the new state, so
//     within a launch exactly one thread touches a given state element.  A decode
//     step consists of heads only: one channel per thread keeps their chains of
//     dependent loads short.
#include "common.h"

#define SC_MAX_L 8

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T* p, float out[VEC]) {
  if (VEC == 8) {
    load8<T>(p, out);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[i] = to_f32<T>(p[i]);
  }
}

template <typename T, int VEC>
__device__ __forceinline__ void store_vec(T* p, const float in[VEC]) {
  if (VEC == 8) {
    store8<T>(p, in);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = from_f32<T>(in[i]);
  }
}

#define SC_TOK 4   // tokens per body thread

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
short_conv_kernel(const T* __restrict__ z, const float* __restrict__ w,
                  const float* __restrict__ bias, float* __restrict__ state,
                  const int* __restrict__ token_seq, const int* __restrict__ seq_start,
                  const int* __restrict__ slot_id, T* __restrict__ y, int width, int L,
                  long long slot_stride, int n_tokens, int body_blocks, int body_total,
                  int head_blocks) {
  const size_t zs = (size_t)3 * width;  // row stride of z
  // the head serves the first `reach` tokens of a portion: those that need the old
  // state, and at least one, so that a step of single tokens needs no body
  const int reach = L > 1 ? L - 1 : 1;

  // The heads come first in the grid: their chain of dependent loads (request, slot,
  // state, inputs) is long, and started last it would stand alone at the kernel's end.
  const int head_total = (int)gridDim.x - body_total;
  if ((int)blockIdx.x >= head_total) {
    // ---- body: tokens t0 .. t0 + SC_TOK - 1, those whose inputs all lie in their portion
    const int bb_ = (int)blockIdx.x - head_total;
    const int t0 = (bb_ / body_blocks) * SC_TOK;
    const int ch = ((bb_ % body_blocks) * blockDim.x + threadIdx.x) * VEC;
    if (ch >= width) return;
    // Every load below is issued before anything is waited for: which of the four
    // tokens are this thread's to write is known only after two dependent lookups
    // (the token's request, that request's first token), and the inputs' addresses do
    // not depend on it.
    int seq_of[SC_TOK];
#pragma unroll
    for (int i = 0; i < SC_TOK; ++i) seq_of[i] = t0 + i < n_tokens ? token_seq[t0 + i] : -1;
    float wt[SC_MAX_L][VEC], c[SC_TOK][VEC];
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
#pragma unroll
      for (int v = 0; v < VEC; ++v) wt[j][v] = 0.f;
#pragma unroll
    for (int j = 0; j < SC_MAX_L; ++j)
      if (j < L) load_vec<float, VEC>(w + (size_t)j * width + ch, wt[j]);
#pragma unroll
    for (int i = 0; i < SC_TOK; ++i)
#pragma unroll
      for (int v = 0; v < VEC; ++v) c[i][v] = bias ? bias[ch + v] : 0.f;
    float cc[SC_TOK][VEC];
#pragma unroll
    for (int i = 0; i < SC_TOK; ++i) {
      const int t = t0 + i < n_tokens ? t0 + i : n_tokens - 1;
      load_vec<T, VEC>(z + (size_t)t * zs + width + ch, cc[i]);
    }
    // row r of the window is token t0 - (L - 1) + r; output i uses rows i .. i + L - 1
#pragma unroll
    for (int r = 0; r < SC_TOK + SC_MAX_L - 1; ++r)
      if (r < SC_TOK + L - 1) {
        int row = t0 - (L - 1) + r;
        row = row < 0 ? 0 : (row >= n_tokens ? n_tokens - 1 : row);   // unused when clamped
        const T* zr = z + (size_t)row * zs;
        float bb[VEC], xx[VEC];
        load_vec<T, VEC>(zr + ch, bb);
        load_vec<T, VEC>(zr + 2 * width + ch, xx);
#pragma unroll
        for (int i = 0; i < SC_TOK; ++i) {
          const int j = r - i;   // the tap with which row r enters output i
          if (j >= 0 && j < SC_MAX_L && j < L) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) c[i][v] = fmaf(wt[j][v], bb[v] * xx[v], c[i][v]);
          }
        }
      }
#pragma unroll
    for (int i = 0; i < SC_TOK; ++i) {
      // mine: the token exists and all its L inputs lie in its own portion
      if (seq_of[i] >= 0 && t0 + i - seq_start[seq_of[i]] >= reach) {
        float o[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) o[v] = cc[i][v] * c[i][v];
        store_vec<T, VEC>(y + (size_t)(t0 + i) * width + ch, o);
      }
    }
    return;
  }

  // ---- head: the outputs that reach into the carried state, then the new state
  const int hb = (int)blockIdx.x;
  const int s = hb / head_blocks;
  const int ch = (hb % head_blocks) * blockDim.x + threadIdx.x;
  if (ch >= width) return;
  const int first = seq_start[s];
  const int t = first;
  const int n = seq_start[s + 1] - first;
  if (n <= 0) return;
  float wt[SC_MAX_L];
#pragma unroll
  for (int j = 0; j < SC_MAX_L; ++j) wt[j] = j < L ? w[(size_t)j * width + ch] : 0.f;
  const float b = bias ? bias[ch] : 0.f;
  auto gate_in = [&](int row) -> float {
    const T* zr = z + (size_t)row * zs;
    return to_f32<T>(zr[ch]) * to_f32<T>(zr[2 * width + ch]);
  };
  auto gate_out = [&](int row, float c) {
    y[(size_t)row * width + ch] = from_f32<T>(to_f32<T>(z[(size_t)row * zs + width + ch]) * c);
  };
  float* st = state + (size_t)slot_id[s] * (size_t)slot_stride + (size_t)ch * L;
  float hist[SC_MAX_L];  // hist[0..L-1]: the last L inputs, oldest first
#pragma unroll
  for (int j = 0; j < SC_MAX_L; ++j) hist[j] = j < L ? st[j] : 0.f;
  const int served = n < reach ? n : reach;  // tokens this thread serves
  for (int i = 0; i < served; ++i) {
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
    gate_out(t + i, c);
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
                             void* y, int dtype, int n_tokens, int n_seqs, int width, int L,
                             long long slot_stride, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || n_seqs <= 0 || n_seqs > n_tokens || width <= 0 || L <= 0 || !z || !w || !state || !token_seq || !seq_start ||
      !slot_id || !y || slot_stride < (long long)width * L)
    return ZA_ERR_ARG;
  if (L > SC_MAX_L) return ZA_ERR_UNSUPPORTED;
  if (dtype != 0 && dtype != 1) return ZA_ERR_UNSUPPORTED;
  const bool vec = width % 8 == 0;   // rows of z and y then start on 16-byte boundaries
  const int per_thread = vec ? 8 : 1;
  const int body_threads = (width + per_thread - 1) / per_thread;
  const int body_blocks = (body_threads + 255) / 256, head_blocks = (width + 255) / 256;
  // a step of single tokens has no body at all
  const long long body_total =
      n_tokens > n_seqs ? (long long)((n_tokens + SC_TOK - 1) / SC_TOK) * body_blocks : 0;
  const long long blocks = body_total + (long long)n_seqs * head_blocks;
  if (blocks > 0x7fffffffLL) return ZA_ERR_UNSUPPORTED;
  dim3 grid((unsigned)blocks), block(256);
#define ZA_SC_LAUNCH(T, VEC)                                                                 \
  hipLaunchKernelGGL((short_conv_kernel<T, VEC>), grid, block, 0, stream, (const T*)z, w,    \
                     bias, state, token_seq, seq_start, slot_id, (T*)y, width, L, slot_stride, \
                     n_tokens, body_blocks, (int)body_total, head_blocks)
  if (dtype == 0) {
    if (vec) ZA_SC_LAUNCH(float, 8); else ZA_SC_LAUNCH(float, 1);
  } else {
    if (vec) ZA_SC_LAUNCH(bf16_t, 8); else ZA_SC_LAUNCH(bf16_t, 1);
  }
#undef ZA_SC_LAUNCH
  return za_launch_status();
}
