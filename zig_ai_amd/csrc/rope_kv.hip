// Per-head RMSNorm of queries and keys, rotary position encoding, and the
// scatter of keys and values into their cache pages: one pass over the fused
// q|k|v projection.
//
// Per (token, head), in 32-bit:
//   q, k:  x <- x * (1/sqrt(mean(x^2) + eps)) * w[head_dim]      (if norm weights are given;
//          before the rotation, never on v: /root/reference/src/transformer/hybrid_attn.zig:371-382)
//   q, k:  for pair p < rotary_dim/2 with angle = position * inv_freq[p]:
//            (a, b) <- (a cos - b sin, a sin + b cos)
//          (/root/reference/src/transformer/rope.zig:40-56); the pair is (p, p + rotary_dim/2)
//          for "half" pairing (the reference's device kernel,
//          /root/reference/src/cuda/layer_kernels.cu:353-365) or (2p, 2p+1) for "adjacent"
//          pairing (rope.zig:46-53).  Elements beyond rotary_dim pass through.
//   k -> cache[page][0][kv_head][offset][head_dim],  slot = page * page_size + offset
//   v -> cache[page][1][kv_head][head_dim][offset]   (turned round: the attention kernels
//        read, for one head-dimension element, consecutive keys side by side)
//   q    -> q_out[token][head][head_dim]
#include "common.h"
#include "rope_math.h"

#define RK_MAX_D 256

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_kv_write_kernel(const T* __restrict__ qkv, const int* __restrict__ positions,
                             const int* __restrict__ slots, const float* __restrict__ q_norm_w,
                             const float* __restrict__ k_norm_w, const float* __restrict__ inv_freq,
                             T* __restrict__ q_out, T* __restrict__ kv_cache, int nh, int nkv, int d,
                             int rot, int adjacent, float eps, int page_size, int write_kv) {
  __shared__ float vec[4][RK_MAX_D];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + wave;  // 0..nh-1: q; then nkv k heads; then nkv v heads
  const int total = nh + 2 * nkv;
  const bool active = head < total;
  const bool is_q = head < nh;
  const bool is_k = !is_q && head < nh + nkv;
  float* s = vec[wave];

  float ss = 0.f;
  if (active) {
    const T* src = qkv + ((size_t)t * total + head) * d;
    for (int i = lane; i < d; i += 64) {
      const float v = to_f32<T>(src[i]);
      s[i] = v;
      ss += v * v;
    }
  }
  ss = wave_sum(ss);
  __syncthreads();
  const float* nw = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
  if (active && nw) {
    const float scale = 1.0f / sqrtf(ss / (float)d + eps);
    for (int i = lane; i < d; i += 64) s[i] = s[i] * scale * nw[i];
  }
  __syncthreads();
  if (active && (is_q || is_k) && rot > 0) {
    const float pos = (float)positions[t];
    const int half = rot / 2;
    for (int p = lane; p < half; p += 64) {
      const int i0 = adjacent ? 2 * p : p;
      const int i1 = adjacent ? 2 * p + 1 : p + half;
      const float angle = pos * inv_freq[p];
      float sn, cs;
      sincosf(angle, &sn, &cs);
      const float a = s[i0], b = s[i1];
      s[i0] = a * cs - b * sn;
      s[i1] = a * sn + b * cs;
    }
  }
  __syncthreads();
  if (!active) return;
  if (is_q) {
    T* dst = q_out + ((size_t)t * nh + head) * d;
    for (int i = lane; i < d; i += 64) dst[i] = from_f32<T>(s[i]);
  } else if (write_kv) {
    const int slot = slots[t];
    if (slot < 0) return;
    const int page = slot / page_size, off = slot % page_size;
    const int kvh = is_k ? head - nh : head - nh - nkv;
    if (is_k) {
      T* dst = kv_cache + ((((size_t)page * 2) * nkv + kvh) * page_size + off) * d;
      for (int i = lane; i < d; i += 64) dst[i] = from_f32<T>(s[i]);
    } else {
      T* dst = kv_cache + (((size_t)page * 2 + 1) * nkv + kvh) * page_size * d + off;
      for (int i = lane; i < d; i += 64) dst[(size_t)i * page_size] = from_f32<T>(s[i]);
    }
  }
}

// The same for head sizes that are powers of two: a block per token, D / 8 lanes per
// head with 16-byte accesses, the token's cosines and sines computed once for all its
// heads, the mean square summed over the head's lanes with lane shuffles.  Half
// pairing needs rotary_dim / 2 to be a multiple of 8, so that a lane's partner
// elements all sit in one other lane.
template <typename T, int D>
__global__ void __launch_bounds__(256)
qk_norm_rope_kv_write_pow2_kernel(const T* __restrict__ qkv, const int* __restrict__ positions,
                                  const int* __restrict__ slots,
                                  const float* __restrict__ q_norm_w,
                                  const float* __restrict__ k_norm_w,
                                  const float* __restrict__ inv_freq, T* __restrict__ q_out,
                                  T* __restrict__ kv_cache, int nh, int nkv, int rot, int adjacent,
                                  float eps, int page_size, int write_kv, int n_tokens,
                                  int value_blocks) {
  constexpr int LPH = D / 8;   // lanes per head
  __shared__ float cs_tab[D / 2], sn_tab[D / 2];
  if ((int)blockIdx.x < value_blocks) {
    // ---- values only, for steps of many tokens: a wave takes eight consecutive tokens
    // and stores, where these lie at eight neighbouring offsets of one page from a
    // multiple of eight on (a stretch of a prompt), each head-dim element's eight
    // values with one 16-byte access (32 bytes in 32-bit) instead of eight 2-byte
    // ones a page row apart.  Other groups (a request's edge, single tokens between
    // prompts) store element by element.
    const int lane = threadIdx.x & 63;
    const int t0 = ((int)blockIdx.x * 4 + ((int)threadIdx.x >> 6)) * 8;   // a wave's 8 tokens
    if (t0 >= n_tokens) return;
    const int total = nh + 2 * nkv;
    int slot[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) slot[j] = t0 + j < n_tokens ? slots[t0 + j] : -1;
    bool side_by_side = page_size % 8 == 0 && slot[0] >= 0 && slot[0] % 8 == 0;
#pragma unroll
    for (int j = 1; j < 8; ++j) side_by_side = side_by_side && slot[j] == slot[0] + j;
    for (int pair = lane; pair < nkv * LPH; pair += 64) {
      const int hv = pair / LPH, e0 = (pair % LPH) * 8;
      float x[8][8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (t0 + j < n_tokens)
          load8<T>(qkv + ((size_t)(t0 + j) * total + nh + nkv + hv) * D + e0, x[j]);
      if (side_by_side) {
        T* dst = kv_cache + (((size_t)(slot[0] / page_size) * 2 + 1) * nkv + hv) * page_size * D +
                 (size_t)e0 * page_size + slot[0] % page_size;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float run[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) run[j] = x[j][i];
          store8<T>(dst + (size_t)i * page_size, run);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (slot[j] >= 0) {
            T* dst = kv_cache +
                     (((size_t)(slot[j] / page_size) * 2 + 1) * nkv + hv) * page_size * D +
                     (size_t)e0 * page_size + slot[j] % page_size;
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[(size_t)i * page_size] = from_f32<T>(x[j][i]);
          }
      }
    }
    return;
  }
  const int t = (int)blockIdx.x - value_blocks;
  const int half = rot / 2;
  const int total = nh + 2 * nkv;
  const int heads_here = value_blocks > 0 ? nh + nkv : total;   // values go their own way
  const int li = threadIdx.x % LPH;
  const int e0 = li * 8;        // this lane's first element of the head
  // this thread's first head is requested before the angles are worked out, and each
  // further head while the one before it is being processed
  float xn[8];
  if ((int)threadIdx.x / LPH < heads_here)
    load8<T>(qkv + ((size_t)t * total + threadIdx.x / LPH) * D + e0, xn);
  if ((int)threadIdx.x < half) {
    float sn, cs;
    rope_angle(positions[t], inv_freq[threadIdx.x], &cs, &sn);
    cs_tab[threadIdx.x] = cs;
    sn_tab[threadIdx.x] = sn;
  }
  __syncthreads();
  for (int head = threadIdx.x / LPH; head < heads_here; head += 256 / LPH) {
    const bool is_q = head < nh;
    const bool is_k = !is_q && head < nh + nkv;
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = xn[i];
    if (head + 256 / LPH < heads_here)
      load8<T>(qkv + ((size_t)t * total + head + 256 / LPH) * D + e0, xn);
    const float* nw = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
    if (nw) {
      // (the decode attention's prologue adds the lanes' sums up in this order too:
      // partners 4 lanes apart first, then 2, then 1)
      float ss = rope_sum_squares8(x);
#pragma unroll
      for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      const float scale = rope_rms_scale(ss, D, eps);
      float w8[8];
      load8<float>(nw + e0, w8);     // two 16-byte loads, not eight of 4 bytes
      rope_scale8(x, scale, w8);
    }
    if ((is_q || is_k) && rot > 0) {
      if (adjacent) {
#pragma unroll
        for (int i = 0; i < 8; i += 2)
          if (e0 + i + 1 < rot) {
            const int p = (e0 + i) / 2;
            const float a = x[i], b = x[i + 1], cs = cs_tab[p], sn = sn_tab[p];
            x[i] = a * cs - b * sn;
            x[i + 1] = a * sn + b * cs;
          }
      } else {
        const bool low = e0 < half, in_rot = e0 < rot;
        const int lane = threadIdx.x & 63;
        const int partner = in_rot ? (low ? lane + half / 8 : lane - half / 8) : lane;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float other = __shfl(x[i], partner, 64);
          if (in_rot) {
            const int p = low ? e0 + i : e0 + i - half;
            const float cs = cs_tab[p], sn = sn_tab[p];
            x[i] = low ? rope_rotate_low(x[i], other, cs, sn) : rope_rotate_high(x[i], other, cs, sn);
          }
        }
      }
    }
    if (is_q) {
      store8<T>(q_out + ((size_t)t * nh + head) * D + e0, x);
    } else if (write_kv) {
      const int slot = slots[t];
      if (slot >= 0) {
        const int page = slot / page_size, off = slot % page_size;
        if (is_k) {
          store8<T>(kv_cache + ((((size_t)page * 2) * nkv + (head - nh)) * page_size + off) * D + e0,
                    x);
        } else {
          T* dst = kv_cache + (((size_t)page * 2 + 1) * nkv + (head - nh - nkv)) * page_size * D +
                   (size_t)e0 * page_size + off;
#pragma unroll
          for (int i = 0; i < 8; ++i) dst[(size_t)i * page_size] = from_f32<T>(x[i]);
        }
      }
    }
  }
}

#define RK_VALUE_BLOCKS_FROM 128   // tokens in a step from which values get blocks of their own

template <typename T>
static bool launch_pow2(const void* qkv, const int* positions, const int* slots,
                        const float* q_norm_w, const float* k_norm_w, const float* inv_freq,
                        void* q_out, void* kv_cache, int n_tokens, int nh, int nkv, int d, int rot,
                        int adjacent, float eps, int page_size, int write_kv,
                        hipStream_t stream) {
  if (!adjacent && (rot / 2) % 8 != 0) return false;
  // many tokens (prompt portions): the values are written by blocks of their own, first
  // in the grid, 32 tokens each
  const int value_blocks = (write_kv && n_tokens >= RK_VALUE_BLOCKS_FROM) ? (n_tokens + 31) / 32 : 0;
#define ZA_RK_LAUNCH(DD)                                                                        \
  hipLaunchKernelGGL((qk_norm_rope_kv_write_pow2_kernel<T, DD>), dim3(n_tokens + value_blocks),  \
                     dim3(256), 0, stream, (const T*)qkv, positions, slots, q_norm_w, k_norm_w,  \
                     inv_freq, (T*)q_out, (T*)kv_cache, nh, nkv, rot, adjacent, eps, page_size,  \
                     write_kv, n_tokens, value_blocks)
  switch (d) {
    case 16: ZA_RK_LAUNCH(16); return true;
    case 32: ZA_RK_LAUNCH(32); return true;
    case 64: ZA_RK_LAUNCH(64); return true;
    case 128: ZA_RK_LAUNCH(128); return true;
    case 256: ZA_RK_LAUNCH(256); return true;
    default: return false;
  }
#undef ZA_RK_LAUNCH
}

extern "C" int za_qk_norm_rope_kv_write(const void* qkv, const int* positions, const int* slots,
                                        const float* q_norm_w, const float* k_norm_w,
                                        const float* inv_freq, void* q_out, void* kv_cache,
                                        int dtype, int n_tokens, int nh, int nkv, int d, int rot,
                                        int adjacent, float eps, int page_size, int write_kv,
                                        hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || nh <= 0 || nkv <= 0 || d <= 0 || !qkv || !positions || !q_out)
    return ZA_ERR_ARG;
  if (d > RK_MAX_D || rot < 0 || rot > d || (rot % 2) != 0) return ZA_ERR_UNSUPPORTED;
  if (rot > 0 && !inv_freq) return ZA_ERR_ARG;
  if (write_kv && (!kv_cache || !slots || page_size <= 0)) return ZA_ERR_ARG;
  if (dtype != 0 && dtype != 1) return ZA_ERR_UNSUPPORTED;
  const bool fast =
      dtype == 0 ? launch_pow2<float>(qkv, positions, slots, q_norm_w, k_norm_w, inv_freq, q_out,
                                      kv_cache, n_tokens, nh, nkv, d, rot, adjacent, eps,
                                      page_size, write_kv, stream)
                 : launch_pow2<bf16_t>(qkv, positions, slots, q_norm_w, k_norm_w, inv_freq, q_out,
                                       kv_cache, n_tokens, nh, nkv, d, rot, adjacent, eps,
                                       page_size, write_kv, stream);
  if (fast) return za_launch_status();
  dim3 grid(n_tokens, (nh + 2 * nkv + 3) / 4), block(256);
  if (dtype == 0) {
    hipLaunchKernelGGL((qk_norm_rope_kv_write_kernel<float>), grid, block, 0, stream,
                       (const float*)qkv, positions, slots, q_norm_w, k_norm_w, inv_freq,
                       (float*)q_out, (float*)kv_cache, nh, nkv, d, rot, adjacent, eps, page_size,
                       write_kv);
  } else if (dtype == 1) {
    hipLaunchKernelGGL((qk_norm_rope_kv_write_kernel<bf16_t>), grid, block, 0, stream,
                       (const bf16_t*)qkv, positions, slots, q_norm_w, k_norm_w, inv_freq,
                       (bf16_t*)q_out, (bf16_t*)kv_cache, nh, nkv, d, rot, adjacent, eps,
                       page_size, write_kv);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
  return za_launch_status();
}
