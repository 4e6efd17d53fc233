// Causal grouped-query attention over paged keys and values, for any mix of
// prompt portions and single decoded tokens in one launch.
//
//   s[t,h,j] = (q[t,h] . k[j,kv(h)]) * scale,  kv(h) = h / (nh / nkv)
//   keys j <= position(t) only, and j > position(t) - window when window > 0
//   softmax over j in 32-bit, streaming: running maximum m and sum l, the
//   accumulator rescaled by exp(m_old - m_new) when the maximum moves
//   o[t,h]   = sum_j p[j] v[j,kv(h)] / l
// (/root/reference/src/transformer/hybrid_attn.zig:553-608 for the dense form,
// /root/reference/src/paged_attention/attention.zig:80-107 and
// /root/reference/src/cuda/paged_attention.cu:190-211 for the streaming form;
// the window has no counterpart there.)
//
// A workgroup serves one work item (up to `count` consecutive query tokens of one
// request) and one key/value head, so a tile of keys staged in LDS is shared by
// every query head of the group and every token of the item.  Rows (token, head)
// are dealt to the four waves; in the score phase a lane owns a key, in the
// value phase it owns head-dimension elements.  Long contexts may be cut into
// `nsplit` ranges of `keys_per_split` keys whose partial (m, l, accumulator) are
// merged by `attention_combine_kernel`; the cut points depend on key positions
// only.
//
// Cache layout: kv[page][0 = keys, 1 = values][kv_head][offset][head_dim].
#include <math.h>

#include "common.h"

#define AT_WAVES 4
#define AT_RPW 8                     // rows per wave, at most
#define AT_MAX_ROWS (AT_WAVES * AT_RPW)
#define AT_MAX_D 256
#define AT_DPL (AT_MAX_D / 64)       // head-dim elements per lane, at most

template <typename T, int KT>
__global__ void __launch_bounds__(256)
paged_attention_kernel(const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kv,
                       const int* __restrict__ block_table, int bt_stride,
                       const int* __restrict__ positions, const int* __restrict__ wi_seq,
                       const int* __restrict__ wi_row0, const int* __restrict__ wi_count,
                       float* __restrict__ part_acc, float* __restrict__ part_ml, int nh, int nkv,
                       int d, int page_size, float scale, int window, int keys_per_split,
                       int nsplit) {
  extern __shared__ float smem[];
  const int ldk = d + 1;
  float* Ks = smem;                       // [KT][d + 1]
  float* Vs = Ks + KT * ldk;              // [KT][d + 1]
  float* Qs = Vs + KT * ldk;              // [AT_MAX_ROWS][d]
  float* Ps = Qs + AT_MAX_ROWS * d;       // [AT_WAVES][64]

  const int item = blockIdx.x, g = blockIdx.y, z = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int G = nh / nkv;
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > AT_MAX_ROWS) count = AT_MAX_ROWS / G;  // the host never asks for more
  const int rows = count * G;
  const int* table = block_table + (size_t)seq * bt_stride;

  const int pos_first = positions[row0];
  const int pos_last = positions[row0 + count - 1];
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int hi = pos_last;  // inclusive
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;
  int tile_first = (lo / KT) * KT;
  if (tile_first < range_lo) tile_first = range_lo;

  // queries of this item, as floats
  for (int idx = tid; idx < rows * d; idx += 256) {
    const int r = idx / d, dd = idx % d;
    const int tok = row0 + r / G, h = g * G + r % G;
    Qs[r * d + dd] = to_f32<T>(q[((size_t)tok * nh + h) * d + dd]);
  }

  float m[AT_RPW], l[AT_RPW], acc[AT_RPW][AT_DPL];
#pragma unroll
  for (int i = 0; i < AT_RPW; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < AT_DPL; ++c) acc[i][c] = 0.f;
  }

  const int vec_per_row = d / 8;
  for (int tile0 = tile_first; tile0 <= range_hi; tile0 += KT) {
    __syncthreads();  // previous tile fully consumed (and Qs written, first time)
    for (int idx = tid; idx < KT * vec_per_row; idx += 256) {
      const int j = idx / vec_per_row, c = (idx % vec_per_row) * 8;
      const int kp = tile0 + j;
      float kx[8], vx[8];
      bool ok = kp >= lo && kp <= range_hi;
      int page = -1;
      if (ok) {
        page = table[kp / page_size];
        ok = page >= 0;
      }
      if (ok) {
        const size_t base = ((((size_t)page * 2) * nkv + g) * page_size + kp % page_size) * d + c;
        const size_t vofs = (size_t)nkv * page_size * d;
        load8<T>(kv + base, kx);
        load8<T>(kv + base + vofs, vx);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) { kx[i] = 0.f; vx[i] = 0.f; }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        Ks[j * ldk + c + i] = kx[i];
        Vs[j * ldk + c + i] = vx[i];
      }
    }
    __syncthreads();

#pragma unroll
    for (int lr = 0; lr < AT_RPW; ++lr) {
      const int r = wave + AT_WAVES * lr;
      if (r < rows) {
        const int pos = positions[row0 + r / G];
        const int kp = tile0 + lane;
        bool valid = lane < KT && kp <= pos && kp <= range_hi && kp >= lo;
        if (window > 0 && kp <= pos - window) valid = false;
        float s = -INFINITY;
        if (lane < KT) {
          const float* qr = Qs + r * d;
          const float* kr = Ks + lane * ldk;
          float dot = 0.f;
          for (int dd = 0; dd < d; ++dd) dot = fmaf(qr[dd], kr[dd], dot);
          if (valid) s = dot * scale;
        }
        const float tmax = wave_max(s);
        const float m_new = fmaxf(m[lr], tmax);
        if (m_new > -INFINITY) {
          const float alpha = expf(m[lr] - m_new);
          const float p = valid ? expf(s - m_new) : 0.f;
          l[lr] = l[lr] * alpha + wave_sum(p);
          m[lr] = m_new;
          __builtin_amdgcn_wave_barrier();
          Ps[wave * 64 + lane] = p;
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int c = 0; c < AT_DPL; ++c) {
            const int dd = lane + 64 * c;
            if (64 * c < d) {
              float a = acc[lr][c] * alpha;
              if (dd < d) {
#pragma unroll 8
                for (int j = 0; j < KT; ++j) a = fmaf(Ps[wave * 64 + j], Vs[j * ldk + dd], a);
              }
              acc[lr][c] = a;
            }
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
  }

#pragma unroll
  for (int lr = 0; lr < AT_RPW; ++lr) {
    const int r = wave + AT_WAVES * lr;
    if (r < rows) {
      const int tok = row0 + r / G, h = g * G + r % G;
      if (nsplit == 1) {
        const float inv = l[lr] > 0.f ? 1.0f / l[lr] : 0.f;
        T* o = out + ((size_t)tok * nh + h) * d;
#pragma unroll
        for (int c = 0; c < AT_DPL; ++c) {
          const int dd = lane + 64 * c;
          if (dd < d) o[dd] = from_f32<T>(acc[lr][c] * inv);
        }
      } else {
        const size_t pidx = ((size_t)tok * nh + h) * nsplit + z;
        float* pa = part_acc + pidx * d;
#pragma unroll
        for (int c = 0; c < AT_DPL; ++c) {
          const int dd = lane + 64 * c;
          if (dd < d) pa[dd] = acc[lr][c];
        }
        if (lane == 0) {
          part_ml[pidx * 2] = m[lr];
          part_ml[pidx * 2 + 1] = l[lr];
        }
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(64)
attention_combine_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                         T* __restrict__ out, int d, int nsplit) {
  const size_t row = blockIdx.x;  // token * nh + head
  const int lane = threadIdx.x;
  float mx = -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, part_ml[(row * nsplit + z) * 2]);
  float total = 0.f;
  float acc[AT_DPL];
#pragma unroll
  for (int c = 0; c < AT_DPL; ++c) acc[c] = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = part_ml[(row * nsplit + z) * 2];
    const float lz = part_ml[(row * nsplit + z) * 2 + 1];
    if (!(mz > -INFINITY)) continue;
    const float w = expf(mz - mx);
    total += lz * w;
    const float* pa = part_acc + (row * nsplit + z) * d;
#pragma unroll
    for (int c = 0; c < AT_DPL; ++c) {
      const int dd = lane + 64 * c;
      if (dd < d) acc[c] = fmaf(pa[dd], w, acc[c]);
    }
  }
  const float inv = total > 0.f ? 1.0f / total : 0.f;
#pragma unroll
  for (int c = 0; c < AT_DPL; ++c) {
    const int dd = lane + 64 * c;
    if (dd < d) out[row * d + dd] = from_f32<T>(acc[c] * inv);
  }
}

template <typename T, int KT>
static int launch_attention(const void* q, void* out, const void* kv, const int* block_table,
                            int bt_stride, const int* positions, const int* wi_seq,
                            const int* wi_row0, const int* wi_count, int n_items, float* part_acc,
                            float* part_ml, int nh, int nkv, int d, int page_size, float scale,
                            int window, int keys_per_split, int nsplit, hipStream_t stream) {
  const size_t shmem =
      ((size_t)2 * KT * (d + 1) + (size_t)AT_MAX_ROWS * d + AT_WAVES * 64) * sizeof(float);
  auto kernel = paged_attention_kernel<T, KT>;
  static size_t allowed = 0;
  if (shmem > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
    allowed = shmem;
  }
  dim3 grid(n_items, nkv, nsplit), block(256);
  hipLaunchKernelGGL(kernel, grid, block, shmem, stream, (const T*)q, (T*)out, (const T*)kv,
                     block_table, bt_stride, positions, wi_seq, wi_row0, wi_count, part_acc,
                     part_ml, nh, nkv, d, page_size, scale, window, keys_per_split, nsplit);
  return za_launch_status();
}

// dtype codes: 0 = float32, 1 = bfloat16
extern "C" int za_paged_attention(const void* q, void* out, const void* kv, const int* block_table,
                                  int bt_stride, const int* positions, const int* wi_seq,
                                  const int* wi_row0, const int* wi_count, int n_items,
                                  int n_tokens, float* part_acc, float* part_ml, int dtype, int nh,
                                  int nkv, int d, int page_size, float scale, int window,
                                  int keys_per_split, int nsplit, hipStream_t stream) {
  if (n_items == 0 || n_tokens == 0) return 0;
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || d <= 0 || page_size <= 0 ||
      bt_stride <= 0 || nsplit < 1 || !q || !out || !kv || !block_table || !positions ||
      !wi_seq || !wi_row0 || !wi_count)
    return ZA_ERR_ARG;
  if (d % 8 != 0 || d > AT_MAX_D || nh / nkv > AT_MAX_ROWS || nkv > 65535 || nsplit > 65535)
    return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  int rc;
#define ZA_AT_ARGS                                                                            \
  q, out, kv, block_table, bt_stride, positions, wi_seq, wi_row0, wi_count, n_items, part_acc, \
      part_ml, nh, nkv, d, page_size, scale, window, keys_per_split, nsplit, stream
  if (dtype == 0) {
    rc = d <= 128 ? launch_attention<float, 64>(ZA_AT_ARGS) : launch_attention<float, 32>(ZA_AT_ARGS);
  } else if (dtype == 1) {
    rc = d <= 128 ? launch_attention<bf16_t, 64>(ZA_AT_ARGS)
                  : launch_attention<bf16_t, 32>(ZA_AT_ARGS);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
#undef ZA_AT_ARGS
  if (rc != 0 || nsplit == 1) return rc;
  dim3 grid((unsigned)((size_t)n_tokens * nh)), block(64);
  if (dtype == 0)
    hipLaunchKernelGGL((attention_combine_kernel<float>), grid, block, 0, stream, part_acc,
                       part_ml, (float*)out, d, nsplit);
  else
    hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), grid, block, 0, stream, part_acc,
                       part_ml, (bf16_t*)out, d, nsplit);
  return za_launch_status();
}
