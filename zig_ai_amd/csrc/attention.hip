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

// ------------------------------------------------------------ matrix-core path
// bfloat16, head_dim 64 or 128, query heads per key/value head dividing 16: the
// same streaming softmax with both products on the matrix cores.
//
// A workgroup serves up to 64 rows (token, head) of one work item and one
// key/value head; each of its four waves owns 16 rows.  Per tile of 64 keys:
//   S^T = K Q^T   (keys as the rows of the first operand, the wave's 16 query rows as
//                  columns; a lane ends up with the scores of ONE query row for 16 keys)
//   p   = exp(S^T * scale - m)  in 32-bit, running maximum and sum kept per lane
//   O^T += V^T P^T  (P^T goes from the accumulator registers straight into the second
//                  operand: the matrix core does not care in which order the 32 keys of
//                  a step are numbered as long as both operands agree, so V^T is stored
//                  in LDS with its keys in the order the accumulator yields them)
// Operand layout of v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k-slots
// (l / 16) * 8 .. + 7 of either operand and receives rows (l / 16) * 4 .. + 3, column
// (l % 16) of the product.
#define AM_KT 64

template <int D>
__global__ void __launch_bounds__(256)
paged_attention_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                            const bf16_t* __restrict__ kv, const int* __restrict__ block_table,
                            int bt_stride, const int* __restrict__ positions,
                            const int* __restrict__ wi_seq, const int* __restrict__ wi_row0,
                            const int* __restrict__ wi_count, int nh, int nkv, int page_size,
                            float scale, int window) {
  constexpr int LDK = D + 8;        // padded rows, in elements
  constexpr int LDV = AM_KT + 8;
  constexpr int KSTEPS = D / 32;    // matrix-core steps over the head dimension
  constexpr int DBLK = D / 16;      // 16-wide blocks of the head dimension
  constexpr int VEC_PER_ROW = D / 8;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[AM_KT * LDK];   // [key][dim]
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D * LDV];       // [dim][key slot]

  const int item = blockIdx.x, gkv = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, grp = lane >> 4;
  const int G = nh / nkv;
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > 64) count = 64 / G;   // the host never asks for more
  const int rows = count * G;
  const int* table = block_table + (size_t)seq * bt_stride;

  const int rr = wave * 16 + r16;
  const bool row_valid = rr < rows;
  const int tok = row0 + (row_valid ? rr / G : 0);
  const int head = gkv * G + (row_valid ? rr % G : 0);
  const int pos_row = row_valid ? positions[tok] : -1;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8_t qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks)
    qf[ks] = row_valid ? *reinterpret_cast<const bf16x8_t*>(
                             q + ((size_t)tok * nh + head) * D + ks * 32 + grp * 8)
                       : zero8;

  const int pos_first = positions[row0];
  const int pos_last = positions[row0 + count - 1];
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int hi = pos_last;
  // what this wave's rows can see at most
  const int wave_first_row = wave * 16;
  const bool wave_active = wave_first_row < rows;
  int wave_last_tok = (wave_first_row + 15) / G;
  if (wave_last_tok > count - 1) wave_last_tok = count - 1;
  const int wave_hi = wave_active ? positions[row0 + wave_last_tok] : -1;

  f32x4_t o[DBLK];
#pragma unroll
  for (int db = 0; db < DBLK; ++db) o[db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const size_t vofs = (size_t)nkv * page_size * D;
  for (int tile0 = (lo / AM_KT) * AM_KT; tile0 <= hi; tile0 += AM_KT) {
    __syncthreads();
    // keys: lanes run along the head dimension (coalesced rows)
#pragma unroll
    for (int v = 0; v < AM_KT * VEC_PER_ROW / 256; ++v) {
      const int idx = tid + v * 256;
      const int j = idx / VEC_PER_ROW, c = (idx % VEC_PER_ROW) * 8;
      const int kp = tile0 + j;
      bf16x8_t kx = zero8;
      if (kp >= lo && kp <= hi) {
        const int page = table[kp / page_size];
        if (page >= 0)
          kx = *reinterpret_cast<const bf16x8_t*>(
              kv + ((((size_t)page * 2) * nkv + gkv) * page_size + kp % page_size) * D + c);
      }
      *reinterpret_cast<bf16x8_t*>(Ks + j * LDK + c) = kx;
    }
    // values, transposed: lanes run along the keys so that the 2-byte stores of one
    // instruction fall side by side
#pragma unroll
    for (int v = 0; v < AM_KT * VEC_PER_ROW / 256; ++v) {
      const int idx = tid + v * 256;
      const int j = idx % AM_KT, c = (idx / AM_KT) * 8;
      const int kp = tile0 + j;
      bf16x8_t vx = zero8;
      if (kp >= lo && kp <= hi) {
        const int page = table[kp / page_size];
        if (page >= 0)
          vx = *reinterpret_cast<const bf16x8_t*>(
              kv + ((((size_t)page * 2) * nkv + gkv) * page_size + kp % page_size) * D + vofs + c);
      }
      // key j of the tile sits in slot: 32-key step, then lane group, then block, then i
      const int slot = (j & 32) + ((j & 15) >> 2) * 8 + ((j >> 4) & 1) * 4 + (j & 3);
#pragma unroll
      for (int e = 0; e < 8; ++e) Vt[(c + e) * LDV + slot] = vx[e];
    }
    __syncthreads();

    if (wave_active && tile0 <= wave_hi) {
      f32x4_t s[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        s[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(
              Ks + (jb * 16 + r16) * LDK + ks * 32 + grp * 8);
          s[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], s[jb], 0, 0, 0);
        }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int kp = tile0 + jb * 16 + grp * 4 + i;
          bool valid = kp <= pos_row && kp >= lo;
          if (window > 0 && kp <= pos_row - window) valid = false;
          const float v = valid ? s[jb][i] * scale : -INFINITY;
          s[jb][i] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m, tmax);
      const float m_use = m_new > -INFINITY ? m_new : 0.f;
      const float alpha = expf(m - m_use);          // m = -inf gives 0
      float psum = 0.f;
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = expf(s[jb][i] - m_use);   // masked scores give 0
          s[jb][i] = p;
          psum += p;
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l = l * alpha + psum;
      m = m_new;
#pragma unroll
      for (int db = 0; db < DBLK; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
      bf16x8_t pf[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pf[kk][i] = (bf16_t)s[2 * kk][i];
          pf[kk][4 + i] = (bf16_t)s[2 * kk + 1][i];
        }
#pragma unroll
      for (int db = 0; db < DBLK; ++db)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
              Vt + (db * 16 + r16) * LDV + kk * 32 + grp * 8);
          o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[kk], o[db], 0, 0, 0);
        }
    }
  }

  if (row_valid) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16_t* dst = out + ((size_t)tok * nh + head) * D;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[db * 16 + grp * 4 + i] = (bf16_t)(o[db][i] * inv);
  }
}

// Decoding on the matrix cores: work items of at most 16 rows (one or a few
// tokens times the query heads of the group), which become the 16 columns of the
// second operand.  The four waves of a workgroup take the key tiles of the
// workgroup's key range in turn and never wait for each other inside the loop:
// keys go from global memory straight into first-operand registers (a lane needs
// 8 consecutive head-dim elements of one key), values are turned through a
// wave-private LDS tile into the key-major order the second product needs.  At the
// end the four partial (m, l, O) are merged in LDS; with `nsplit` > 1 the merged
// partial goes to `attention_combine_kernel` like those of the plain kernel.
template <int D>
__global__ void __launch_bounds__(256)
paged_attention_decode_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                                   const bf16_t* __restrict__ kv,
                                   const int* __restrict__ block_table, int bt_stride,
                                   const int* __restrict__ positions,
                                   const int* __restrict__ wi_seq, const int* __restrict__ wi_row0,
                                   const int* __restrict__ wi_count, float* __restrict__ part_acc,
                                   float* __restrict__ part_ml, int nh, int nkv, int page_size,
                                   float scale, int window, int keys_per_split, int nsplit) {
  constexpr int LDV = AM_KT + 8;
  constexpr int KSTEPS = D / 32;
  constexpr int DBLK = D / 16;
  constexpr int VEC_PER_ROW = D / 8;
  __shared__ __attribute__((aligned(16))) bf16_t Vt_all[4 * D * LDV];   // [wave][dim][key slot]
  __shared__ float mg_m[4][16], mg_l[4][16];
  __shared__ float mg_o[4][DBLK][64][4];

  const int item = blockIdx.x, gkv = blockIdx.y, z = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, grp = lane >> 4;
  const int G = nh / nkv;
  // without work-item arrays item i is request i's single token (a pure decode step)
  const int seq = wi_seq ? wi_seq[item] : item;
  const int row0 = wi_seq ? wi_row0[item] : item;
  int count = wi_seq ? wi_count[item] : 1;
  if (count * G > 16) count = 16 / G;   // the host never asks for more
  const int rows = count * G;
  const int* table = block_table + (size_t)seq * bt_stride;
  bf16_t* Vt = Vt_all + wave * D * LDV;

  const bool row_valid = r16 < rows;
  const int tok = row0 + (row_valid ? r16 / G : 0);
  const int head = gkv * G + (row_valid ? r16 % G : 0);
  const int pos_row = row_valid ? positions[tok] : -1;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8_t qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks)
    qf[ks] = row_valid ? *reinterpret_cast<const bf16x8_t*>(
                             q + ((size_t)tok * nh + head) * D + ks * 32 + grp * 8)
                       : zero8;

  const int pos_first = positions[row0];
  const int pos_last = positions[row0 + count - 1];
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int hi = pos_last;
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;
  int tile_first = (lo / AM_KT) * AM_KT;
  if (tile_first < range_lo) tile_first = range_lo;

  f32x4_t o[DBLK];
#pragma unroll
  for (int db = 0; db < DBLK; ++db) o[db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const size_t vofs = (size_t)nkv * page_size * D;

  // One tile's keys (first-operand fragments) and values (rows along the head
  // dimension, lane = key) in registers; the next tile is fetched while this one is
  // being computed.
  bf16x8_t kf[4][KSTEPS], vx[VEC_PER_ROW];
  // The block-table entries are read whether or not the key turns out to be in
  // range (unused entries hold -1), so that these loads do not wait for the
  // positions the range is computed from.
  const int last_entry = bt_stride - 1;
  auto fetch = [&](int tile0, bf16x8_t (&kfr)[4][KSTEPS], bf16x8_t (&vxr)[VEC_PER_ROW]) {
    int kpage[4];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const int e = (tile0 + jb * 16 + r16) / page_size;
      kpage[jb] = table[e < last_entry ? e : last_entry];
    }
    const int ve = (tile0 + lane) / page_size;
    const int vpage = table[ve < last_entry ? ve : last_entry];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const int kp = tile0 + jb * 16 + r16;
      const bf16_t* krow = nullptr;
      if (kp >= lo && kp <= range_hi && kpage[jb] >= 0)
        krow = kv + ((((size_t)kpage[jb] * 2) * nkv + gkv) * page_size + kp % page_size) * D;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        kfr[jb][ks] = krow ? *reinterpret_cast<const bf16x8_t*>(krow + ks * 32 + grp * 8) : zero8;
    }
    const int kp = tile0 + lane;
    const bf16_t* vrow = nullptr;
    if (kp >= lo && kp <= range_hi && vpage >= 0)
      vrow = kv + ((((size_t)vpage * 2) * nkv + gkv) * page_size + kp % page_size) * D + vofs;
#pragma unroll
    for (int v = 0; v < VEC_PER_ROW; ++v)
      vxr[v] = vrow ? *reinterpret_cast<const bf16x8_t*>(vrow + v * 8) : zero8;
  };

  int tile0 = tile_first + wave * AM_KT;
  if (tile0 <= range_hi) fetch(tile0, kf, vx);
  for (; tile0 <= range_hi; tile0 += 4 * AM_KT) {
    bf16x8_t kfn[4][KSTEPS], vxn[VEC_PER_ROW];
    const int next = tile0 + 4 * AM_KT;
    if (next <= range_hi) fetch(next, kfn, vxn);

    f32x4_t s[4];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      s[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        s[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[jb][ks], qf[ks], s[jb], 0, 0, 0);
    }
    // values into this wave's LDS tile, key-major (lane = key j of the tile)
    {
      const int j = lane;
      const int slot = (j & 32) + ((j & 15) >> 2) * 8 + ((j >> 4) & 1) * 4 + (j & 3);
#pragma unroll
      for (int v = 0; v < VEC_PER_ROW; ++v)
#pragma unroll
        for (int e = 0; e < 8; ++e) Vt[(v * 8 + e) * LDV + slot] = vx[v][e];
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kp = tile0 + jb * 16 + grp * 4 + i;
        bool valid = kp <= pos_row && kp >= lo && kp <= range_hi;
        if (window > 0 && kp <= pos_row - window) valid = false;
        const float v = valid ? s[jb][i] * scale : -INFINITY;
        s[jb][i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m, tmax);
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float alpha = expf(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = expf(s[jb][i] - m_use);
        s[jb][i] = p;
        psum += p;
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
    bf16x8_t pf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pf[kk][i] = (bf16_t)s[2 * kk][i];
        pf[kk][4 + i] = (bf16_t)s[2 * kk + 1][i];
      }
    __builtin_amdgcn_wave_barrier();   // this wave's stores to Vt precede its loads below
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
            Vt + (db * 16 + r16) * LDV + kk * 32 + grp * 8);
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[kk], o[db], 0, 0, 0);
      }
    __builtin_amdgcn_wave_barrier();   // and those loads precede the next tile's stores
    if (next <= range_hi) {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) kf[jb][ks] = kfn[jb][ks];
#pragma unroll
      for (int v = 0; v < VEC_PER_ROW; ++v) vx[v] = vxn[v];
    }
  }

  // merge the four waves' partial results
  if (grp == 0) { mg_m[wave][r16] = m; mg_l[wave][r16] = l; }
#pragma unroll
  for (int db = 0; db < DBLK; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) mg_o[wave][db][lane][i] = o[db][i];
  __syncthreads();
  if (wave == 0 && row_valid) {
    float mx = mg_m[0][r16];
#pragma unroll
    for (int w = 1; w < 4; ++w) mx = fmaxf(mx, mg_m[w][r16]);
    const float mu = mx > -INFINITY ? mx : 0.f;
    float wgt[4], total = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      wgt[w] = expf(mg_m[w][r16] - mu);
      total += mg_l[w][r16] * wgt[w];
    }
    const size_t orow = (size_t)tok * nh + head;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) acc = fmaf(mg_o[w][db][lane][i], wgt[w], acc);
        const int dim = db * 16 + grp * 4 + i;
        if (nsplit == 1)
          out[orow * D + dim] = (bf16_t)(total > 0.f ? acc / total : 0.f);
        else
          part_acc[(orow * nsplit + z) * D + dim] = acc;
      }
    if (nsplit > 1 && grp == 0) {
      part_ml[(orow * nsplit + z) * 2] = mx;
      part_ml[(orow * nsplit + z) * 2 + 1] = total;
    }
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

// Matrix-core variant: bfloat16 only, head_dim 64 or 128, (nh / nkv) dividing 16, work
// items of at most 64 / (nh / nkv) query rows.  Returns ZA_ERR_UNSUPPORTED otherwise.
extern "C" int za_paged_attention_mfma(const void* q, void* out, const void* kv,
                                       const int* block_table, int bt_stride,
                                       const int* positions, const int* wi_seq,
                                       const int* wi_row0, const int* wi_count, int n_items,
                                       int nh, int nkv, int d, int page_size, float scale,
                                       int window, hipStream_t stream) {
  if (n_items == 0) return 0;
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || page_size <= 0 || bt_stride <= 0 ||
      !q || !out || !kv || !block_table || !positions || !wi_seq || !wi_row0 || !wi_count)
    return ZA_ERR_ARG;
  const int G = nh / nkv;
  if ((d != 64 && d != 128) || G > 16 || 16 % G != 0 || nkv > 65535) return ZA_ERR_UNSUPPORTED;
  dim3 grid(n_items, nkv), block(256);
  if (d == 64)
    hipLaunchKernelGGL((paged_attention_mfma_kernel<64>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, nh, nkv, page_size, scale, window);
  else
    hipLaunchKernelGGL((paged_attention_mfma_kernel<128>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, nh, nkv, page_size, scale, window);
  return za_launch_status();
}

// Matrix-core decode variant: bfloat16, head_dim 64 or 128, work items of at most
// 16 / (nh / nkv) query rows (nh / nkv dividing 16), contexts optionally cut as in
// za_paged_attention (the partial results are merged by the same combine kernel).
extern "C" int za_paged_attention_decode_mfma(const void* q, void* out, const void* kv,
                                              const int* block_table, int bt_stride,
                                              const int* positions, const int* wi_seq,
                                              const int* wi_row0, const int* wi_count,
                                              int n_items, int n_tokens, float* part_acc,
                                              float* part_ml, int nh, int nkv, int d,
                                              int page_size, float scale, int window,
                                              int keys_per_split, int nsplit,
                                              hipStream_t stream) {
  if (n_items == 0 || n_tokens == 0) return 0;
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || page_size <= 0 || bt_stride <= 0 ||
      nsplit < 1 || !q || !out || !kv || !block_table || !positions)
    return ZA_ERR_ARG;
  if (wi_seq && (!wi_row0 || !wi_count)) return ZA_ERR_ARG;
  if (!wi_seq && n_items != n_tokens) return ZA_ERR_ARG;   // identity items: one token each
  const int G = nh / nkv;
  if ((d != 64 && d != 128) || G > 16 || 16 % G != 0 || nkv > 65535 || nsplit > 65535)
    return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  dim3 grid(n_items, nkv, nsplit), block(256);
  if (d == 64) {
    hipLaunchKernelGGL((paged_attention_decode_mfma_kernel<64>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, part_acc, part_ml, nh, nkv,
                       page_size, scale, window, keys_per_split, nsplit);
  } else {
    hipLaunchKernelGGL((paged_attention_decode_mfma_kernel<128>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, part_acc, part_ml, nh, nkv,
                       page_size, scale, window, keys_per_split, nsplit);
  }
  int rc = za_launch_status();
  if (rc != 0 || nsplit == 1) return rc;
  dim3 cgrid((unsigned)((size_t)n_tokens * nh)), cblock(64);
  hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), cgrid, cblock, 0, stream, part_acc,
                     part_ml, (bf16_t*)out, d, nsplit);
  return za_launch_status();
}
