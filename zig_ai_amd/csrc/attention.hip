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
// Cache layout, per page: keys as [kv_head][offset][head_dim], then values turned
// round as [kv_head][head_dim][offset].  The second product wants, for one
// head-dimension element, consecutive keys side by side; stored this way the
// matrix-core kernels fetch their value operands with plain 8-byte loads.
#include <math.h>

#include "common.h"
#include "rope_math.h"

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
      float kx[8];
      bool ok = kp >= lo && kp <= range_hi;
      int page = -1;
      if (ok) {
        page = table[kp / page_size];
        ok = page >= 0;
      }
      if (ok) {
        load8<T>(kv + ((((size_t)page * 2) * nkv + g) * page_size + kp % page_size) * d + c, kx);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) kx[i] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) Ks[j * ldk + c + i] = kx[i];
    }
    {
      // values: a thread keeps one key of the tile (256 is a multiple of KT) and walks
      // the head dimension, so the lanes of a wave read consecutive offsets of a page
      const int j = tid % KT;
      const int kp = tile0 + j;
      const T* vsrc = nullptr;
      if (kp >= lo && kp <= range_hi) {
        const int page = table[kp / page_size];
        if (page >= 0)
          vsrc = kv + (((size_t)page * 2 + 1) * nkv + g) * page_size * d + kp % page_size;
      }
      for (int dd = tid / KT; dd < d; dd += 256 / KT)
        Vs[j * ldk + dd] = vsrc ? to_f32<T>(vsrc[(size_t)dd * page_size]) : 0.f;
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

// `base2`: the partial maxima are whole numbers on the base-2 scale (what the matrix-core
// kernels keep), so a partial result's weight 2^(m_z - m) is an exact power of two.
template <typename T>
__global__ void __launch_bounds__(64)
attention_combine_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                         T* __restrict__ out, int d, int nsplit, int base2) {
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
    const float w = base2 ? ldexpf(1.0f, (int)(mz - mx)) : expf(mz - mx);
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
// bfloat16, head_dim 64 or 128, page sizes that are multiples of 4: the same
// streaming softmax with both products on the matrix cores.
//
// A workgroup serves up to 128 rows (token, head) of one work item and one
// key/value head; each of its eight waves owns 16 rows.  (Waves of 32 rows would read
// LDS half as often, but need so many registers that a SIMD holds one wave only, and
// the kernel is bound by vector instructions and their waits, not by LDS: measured,
// eight light waves are faster.)  Per tile of 64 keys:
//   S^T = K Q^T   (keys as the rows of the first operand, 16 query rows as columns; a
//                  lane ends up with the scores of ONE query row for 16 keys)
//   p   = 2^(S^T * scale * log2(e) - m)  in 32-bit, running maximum per lane; p is rounded
//                  to bfloat16 for the second product, and the sum that normalises the
//                  result is the sum of those rounded values (so the weights that reach
//                  the values add up to one), taken by the matrix core as well;
//                  m is the running maximum ROUNDED UP TO A WHOLE NUMBER, so every
//                  rescaling factor 2^(m_old - m_new) is an exact power of two: the
//                  probabilities' rounding to bfloat16 for the second product is then the
//                  same whatever the order of tiles, ranges and waves (scaling by a power
//                  of two commutes with rounding), and a row's result does not depend on
//                  how its keys were cut beyond the order of 32-bit additions
//   O^T += V^T P^T  (P^T goes from the accumulator registers straight into the second
//                  operand: the matrix core does not care in which order the 32 keys of
//                  a step are numbered as long as both operands agree, so V^T is stored
//                  in LDS with its keys in the order the accumulator yields them)
// The tiles go through two LDS buffers: while a tile is being computed the next one is
// on its way from memory into registers, and the page numbers of the one after that
// are being read.  Every tile issues the same loads, unconditionally.
// Operand layout of v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k-slots
// (l / 16) * 8 .. + 7 of either operand and receives rows (l / 16) * 4 .. + 3, column
// (l % 16) of the product.
#define AM_KT 64       // keys of a tile in the decode kernel (the prefill kernel: 64 or 128)
#define AM_ROWS 128
#define ZA_DECODE_WIDE_BELOW 384   // workgroups: up to here the decode kernel runs eight waves


// A query row's scores for a tile are spread over the four lanes l, l ^ 16, l ^ 32,
// l ^ 48.  The swap instructions exchange 16-lane rows (odd rows of the first operand
// with even rows of the second) and 32-lane halves between two registers; fed the
// same value twice they leave in each lane its own value and its partner's, in one
// vector instruction each and without a trip through LDS.
__device__ __forceinline__ float quad_max(float x) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false,
                                                  false);
  const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(y), __float_as_uint(y), false,
                                                  false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false,
                                                  false);
  const float y = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(y), __float_as_uint(y), false,
                                                  false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Key position -> block-table entry and offset in the page.  Page sizes are powers of
// two nearly always: `shift` is then log2(page_size) and the division (some thirty
// instructions, several times per tile) becomes a shift; otherwise `shift` is -1.
__device__ __forceinline__ int page_shift_of(int page_size) {
  return (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;
}
__device__ __forceinline__ int page_entry(int kp, int page_size, int shift) {
  return shift >= 0 ? kp >> shift : kp / page_size;
}
__device__ __forceinline__ int page_offset(int kp, int page_size, int shift) {
  return shift >= 0 ? kp & (page_size - 1) : kp % page_size;
}

template <int D, int NW, int NS, int KT>
__global__ void __launch_bounds__(NW * 64)
paged_attention_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                            const bf16_t* __restrict__ kv, const int* __restrict__ block_table,
                            int bt_stride, const int* __restrict__ positions,
                            const int* __restrict__ wi_seq, const int* __restrict__ wi_row0,
                            const int* __restrict__ wi_count, int n_items,
                            float* __restrict__ part_acc, float* __restrict__ part_ml, int nh,
                            int nkv, int page_size, float scale_log2e, int window,
                            int keys_per_split, int nsplit) {
  constexpr int LDK = D + 8;        // padded rows, in elements
  constexpr int LDV = KT + 8;
  constexpr int KSTEPS = D / 32;    // matrix-core steps over the head dimension
  constexpr int DBLK = D / 16;      // 16-wide blocks of the head dimension
  constexpr int VEC_PER_ROW = D / 8;
  constexpr int NT = NW * 64;                      // threads
  constexpr int KVEC = KT * VEC_PER_ROW / NT;   // 16-byte pieces of a key tile per thread
  constexpr int VVEC = D * (KT / 4) / NT;       // 8-byte pieces of a value tile per thread
  constexpr int KROWS = NT / VEC_PER_ROW;          // keys between a thread's pieces
  constexpr int JB = KT / 16;                      // blocks of 16 keys in a tile
  constexpr int KK = KT / 32;                      // matrix-core steps over a tile's keys
  constexpr int VRUNS = KT / 4;                    // runs of 4 keys in a tile
  static_assert(NW * NS * 16 == AM_ROWS && KVEC >= 1 && VVEC >= 1 && (KT == 64 || KT == 128),
                "tile shape");
  extern __shared__ __attribute__((aligned(16))) unsigned char am_smem[];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(am_smem);   // [2][key][dim]
  bf16_t* Vt = Ks + 2 * KT * LDK;                 // [2][dim][key slot]

  const int gkv = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, grp = lane >> 4;
  const int G = nh / nkv;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int last_entry = bt_stride - 1;
  const int ps_shift = page_shift_of(page_size);

  // The work of an item grows with its place in a prompt.  The second half of the grid
  // takes its items in descending order, so that workgroups that start together (and
  // share a compute unit) weigh about the same in pairs.
  int item = blockIdx.y;
  {
    const int half = n_items / 2;
    if (item >= half) item = n_items - 1 - (item - half);
  }
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > AM_ROWS) count = AM_ROWS / G;   // the host never asks for more
  const int rows = count * G;
  const int* table = block_table + (size_t)seq * bt_stride;

  int tok[NS], head[NS], pos_row[NS];
  bool row_valid[NS];
  bf16x8_t qf[NS][KSTEPS];
#pragma unroll
  for (int c = 0; c < NS; ++c) {
    const int rr = wave * (NS * 16) + c * 16 + r16;
    row_valid[c] = rr < rows;
    tok[c] = row0 + (row_valid[c] ? rr / G : 0);
    head[c] = gkv * G + (row_valid[c] ? rr % G : 0);
    pos_row[c] = row_valid[c] ? positions[tok[c]] : -1;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      qf[c][ks] = row_valid[c] ? *reinterpret_cast<const bf16x8_t*>(
                                     q + ((size_t)tok[c] * nh + head[c]) * D + ks * 32 + grp * 8)
                               : zero8;
  }

  const int pos_first = positions[row0];
  const int pos_last = positions[row0 + count - 1];
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  // with nsplit > 1 this workgroup serves the keys of one range only (ranges are
  // multiples of the tile, so a tile lies in one range); its partial result is
  // merged with the others' by attention_combine_kernel
  const int z = blockIdx.z;
  int hi = pos_last;
  if (nsplit > 1 && (z + 1) * keys_per_split - 1 < hi) hi = (z + 1) * keys_per_split - 1;
  // what this wave's rows can see
  const int wave_first_row = wave * (NS * 16);
  const bool wave_active = wave_first_row < rows;
  const bool wave_full = wave_first_row + NS * 16 <= rows;
  int wave_last_tok = (wave_first_row + NS * 16 - 1) / G;
  if (wave_last_tok > count - 1) wave_last_tok = count - 1;
  const int wave_hi = wave_active ? positions[row0 + wave_last_tok] : -1;
  const int wave_lo = wave_active ? positions[row0 + wave_first_row / G] : 0;

  f32x4_t o[NS][DBLK], lsum[NS];
  float m[NS];
  bf16x8_t ones8;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones8[i] = (bf16_t)1.0f;
#pragma unroll
  for (int c = 0; c < NS; ++c) {
    m[c] = -INFINITY;
    lsum[c] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < DBLK; ++db) o[c][db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // This thread's pieces of a tile: KVEC 16-byte runs along the head dimension of keys
  // krow0 + v * KROWS, and VVEC 8-byte runs of 4 consecutive keys (run vkr of the
  // tile) for head-dimension elements vdd0 + v * (NT / 16).  What does not change from
  // tile to tile is folded into two base pointers.
  const int krow0 = tid / VEC_PER_ROW, vkr = tid & (VRUNS - 1), vdd0 = tid / VRUNS;
  // (elements of one page, keys and values of all heads: below 2^32, the host checks;
  // page * stride is then ONE 32 x 32 -> 64-bit multiply-add per load)
  const unsigned page_stride = 2u * (unsigned)nkv * (unsigned)page_size * (unsigned)D;
  const bf16_t* kbase = kv + (size_t)gkv * page_size * D + (tid % VEC_PER_ROW) * 8;
  const bf16_t* vbase = kv + ((size_t)nkv + gkv) * page_size * D + (size_t)vdd0 * page_size;
  const int vstep = (NT / VRUNS) * page_size;   // elements between a thread's value pieces

  int kpg[KVEC], vpg;
  bf16x8_t kreg[KVEC];
  bf16x4_t vreg[VVEC];
  auto load_pages = [&](int tile0) {
#pragma unroll
    for (int v = 0; v < KVEC; ++v) {
      const int e = page_entry(tile0 + krow0 + v * KROWS, page_size, ps_shift);
      kpg[v] = table[e < last_entry ? e : last_entry];
    }
    const int e = page_entry(tile0 + vkr * 4, page_size, ps_shift);
    vpg = table[e < last_entry ? e : last_entry];
  };
  // Loads never leave the pool: an unused table entry (-1) reads page 0 instead, and
  // tiles beyond the last one are fetched like any other.  A key that must not count is
  // masked in the scores, whatever its row holds; its values are cleared on their way
  // into LDS, since 0 * (not a number) would not be 0.
  auto load_data = [&](int tile0) {
#pragma unroll
    for (int v = 0; v < KVEC; ++v) {
      const int off = page_offset(tile0 + krow0 + v * KROWS, page_size, ps_shift);
      const unsigned page = kpg[v] < 0 ? 0u : (unsigned)kpg[v];
      kreg[v] = *reinterpret_cast<const bf16x8_t*>(kbase + ((size_t)page * page_stride + (unsigned)(off * D)));
    }
    const int off = page_offset(tile0 + vkr * 4, page_size, ps_shift);
    const unsigned page = vpg < 0 ? 0u : (unsigned)vpg;
    const bf16_t* src = vbase + ((size_t)page * page_stride + (unsigned)off);
#pragma unroll
    for (int v = 0; v < VVEC; ++v)
      vreg[v] = *reinterpret_cast<const bf16x4_t*>(src + v * vstep);
  };
  // keys jb * 16 + g4 * 4 .. + 3 of the tile sit in slots: 32-key step, then lane group,
  // then block
  const int vslot = (vkr >> 3) * 32 + (vkr & 3) * 8 + ((vkr >> 2) & 1) * 4;
  auto store_tile = [&](int buf, int tile0) {
    bf16_t* ks = Ks + buf * KT * LDK;
    bf16_t* vt = Vt + buf * D * LDV;
#pragma unroll
    for (int v = 0; v < KVEC; ++v)
      *reinterpret_cast<bf16x8_t*>(ks + (krow0 + v * KROWS) * LDK + (tid % VEC_PER_ROW) * 8) =
          kreg[v];
    const int kp = tile0 + vkr * 4;
    const bool edge_tile = tile0 < lo || tile0 + KT - 1 > hi;   // the same for all threads
#pragma unroll
    for (int v = 0; v < VVEC; ++v) {
      bf16x4_t x = vreg[v];
      if (edge_tile) {
        // keys outside [lo, hi] (pages that are not there lie outside it too)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (kp + e < lo || kp + e > hi) x[e] = (bf16_t)0.f;
      }
      *reinterpret_cast<bf16x4_t*>(vt + (vdd0 + v * (NT / VRUNS)) * LDV + vslot) = x;
    }
  };

  int tile_first = (lo / KT) * KT;
  if (nsplit > 1 && z * keys_per_split > tile_first) tile_first = z * keys_per_split;
  const int n_tiles = hi >= tile_first ? (hi - tile_first) / KT + 1 : 0;   // 0: an empty range
  load_pages(tile_first);
  load_data(tile_first);
  load_pages(tile_first + KT);
  store_tile(0, tile_first);
  __syncthreads();

  for (int t = 0; t < n_tiles; ++t) {
    const int tile0 = tile_first + t * KT;
    const int buf = t & 1;
    load_data(tile0 + KT);
    load_pages(tile0 + 2 * KT);

    bool wave_sees = wave_active && tile0 <= wave_hi;
    if (window > 0 && tile0 + KT - 1 <= wave_lo - window) wave_sees = false;
    if (wave_sees) {
      const bf16_t* ks = Ks + buf * KT * LDK;
      const bf16_t* vt = Vt + buf * D * LDV;
      f32x4_t s[NS][JB];
#pragma unroll
      for (int jb = 0; jb < JB; ++jb) {
#pragma unroll
        for (int c = 0; c < NS; ++c) s[c][jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks_ = 0; ks_ < KSTEPS; ++ks_) {
          const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(
              ks + (jb * 16 + r16) * LDK + ks_ * 32 + grp * 8);
#pragma unroll
          for (int c = 0; c < NS; ++c)
            s[c][jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c][ks_], s[c][jb], 0, 0, 0);
        }
      }
      // a tile every key of which counts for every row of the wave needs no mask
      const bool needs_mask = !wave_full || tile0 + KT - 1 > wave_lo || tile0 < lo ||
                              tile0 + KT - 1 > hi || (window > 0 && tile0 <= wave_hi - window);
      bf16x8_t pf[NS][KK];
#pragma unroll
      for (int c = 0; c < NS; ++c) {
        if (needs_mask) {
          // key jb * 16 + grp * 4 + i of the tile counts for this lane's row if it lies in
          // [first, last]; both bounds are taken relative to the lane's own keys once, so
          // that an element costs two comparisons with constants
          int last = pos_row[c] < hi ? pos_row[c] : hi;
          int first = lo;
          if (window > 0 && pos_row[c] - window + 1 > first) first = pos_row[c] - window + 1;
          last -= tile0 + grp * 4;
          first -= tile0 + grp * 4;
          const bool below = __any(first > 0);   // does any lane have keys before its first?
#pragma unroll
          for (int jb = 0; jb < JB; ++jb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              bool valid = jb * 16 + i <= last;
              if (below) valid = valid && jb * 16 + i >= first;
              if (!valid) s[c][jb][i] = -INFINITY;
            }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int jb = 0; jb < JB; ++jb)
#pragma unroll
          for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, s[c][jb][i]);
        tmax = quad_max(tmax);
        const float m_new = fmaxf(m[c], ceilf(tmax * scale_log2e));   // the factor is positive
        const float m_use = m_new > -INFINITY ? m_new : 0.f;
        // (nothing is accumulated yet while m is -inf: any finite factor does)
        const float alpha = m[c] > -INFINITY ? ldexpf(1.0f, (int)(m[c] - m_use)) : 1.0f;
#pragma unroll
        for (int jb = 0; jb < JB; ++jb)
#pragma unroll
          for (int i = 0; i < 4; ++i)   // masked scores (-inf) give 0
            s[c][jb][i] = __builtin_amdgcn_exp2f(fmaf(s[c][jb][i], scale_log2e, -m_use));
        m[c] = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int i = 0; i < 4; ++i) lsum[c][i] *= alpha;
#pragma unroll
          for (int db = 0; db < DBLK; ++db)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[c][db][i] *= alpha;
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            pf[c][kk][i] = (bf16_t)s[c][2 * kk][i];
            pf[c][kk][4 + i] = (bf16_t)s[c][2 * kk + 1][i];
          }
          // the row's sum of the ROUNDED probabilities, by the matrix core (a first operand
          // of ones): every one of the accumulator's four values is the sum over the 32
          // keys of the step for the lane's query row, all four lane groups' keys included
          lsum[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones8, pf[c][kk], lsum[c], 0, 0, 0);
        }
      }
#pragma unroll
      for (int db = 0; db < DBLK; ++db)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
              vt + (db * 16 + r16) * LDV + kk * 32 + grp * 8);
#pragma unroll
          for (int c = 0; c < NS; ++c)
            o[c][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c][kk], o[c][db], 0, 0, 0);
        }
    }
    if (t + 1 < n_tiles) store_tile(buf ^ 1, tile0 + KT);
    __syncthreads();
  }

#pragma unroll
  for (int c = 0; c < NS; ++c)
    if (row_valid[c]) {
      const size_t orow = (size_t)tok[c] * nh + head[c];
      if (nsplit > 1) {
        // unnormalised accumulator, and (maximum, sum), the maximum on the base-2 scale
        float* pa = part_acc + (orow * nsplit + z) * D;
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
          *reinterpret_cast<f32x4_t*>(pa + db * 16 + grp * 4) = o[c][db];
        if (grp == 0) {
          part_ml[(orow * nsplit + z) * 2] = m[c];
          part_ml[(orow * nsplit + z) * 2 + 1] = lsum[c][0];
        }
        continue;
      }
      const float inv = lsum[c][0] > 0.f ? 1.0f / lsum[c][0] : 0.f;
      bf16_t* dst = out + orow * D;
#pragma unroll
      for (int db = 0; db < DBLK; ++db) {
        bf16x4_t ov;
#pragma unroll
        for (int i = 0; i < 4; ++i) ov[i] = (bf16_t)(o[c][db][i] * inv);
        *reinterpret_cast<bf16x4_t*>(dst + db * 16 + grp * 4) = ov;
      }
    }
}

// Decoding on the matrix cores: work items of at most 16 rows (one or a few
// tokens times the query heads of the group), which become the 16 columns of the
// second operand.  The waves of a workgroup (NWV: four or eight) take the key tiles of the
// workgroup's key range in turn and never wait for each other inside the loop:
// keys go from global memory straight into first-operand registers (a lane needs
// 8 consecutive head-dim elements of one key), and so do the values (a lane needs,
// for one head-dim element, 8 consecutive keys, which the cache holds side by
// side).  At the end the waves' partial (m, l, O) are merged in LDS; with
// `nsplit` > 1 the merged partial goes to `attention_combine_kernel` like those of
// the plain kernel.
// ROPE: the kernel prepares its token's queries, key and value itself, from the step's fused
// q|k|v projection: per-head RMSNorm of q and k, the rotation (half pairing over the whole
// head), with rope_math.h's expressions and the order of additions of
// qk_norm_rope_kv_write_pow2_kernel, so the bits are those of that kernel followed by this
// one.  Every workgroup of a (request, key/value head) works the key out; the wave whose
// tile holds the token's own position puts key and value into its fragments (the cache does
// not hold them yet) and stores them to the cache for the steps to come.  One token a
// work item only.
struct DecodeRope {
  const bf16_t* qkv;        // [tokens][nh + 2 nkv][D]
  const int* slots;         // a token's place in the cache (page * page_size + offset), -1: none
  const float* q_norm_w;    // [D] each, or null: no norm
  const float* k_norm_w;
  const float* inv_freq;    // [D / 2]
  bf16_t* kv_write;         // the cache, to store the token's key and value
  float eps;
  int write_kv;
};

template <int D, int NWV, bool ROPE>
__global__ void __launch_bounds__(NWV * 64)
paged_attention_decode_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                                   const bf16_t* kv,
                                   const int* __restrict__ block_table, int bt_stride,
                                   const int* __restrict__ positions,
                                   const int* __restrict__ wi_seq, const int* __restrict__ wi_row0,
                                   const int* __restrict__ wi_count, float* __restrict__ part_acc,
                                   float* __restrict__ part_ml, int nh, int nkv, int page_size,
                                   float scale_log2e, int window, int keys_per_split, int nsplit,
                                   DecodeRope rope) {
  constexpr int KSTEPS = D / 32;
  constexpr int DBLK = D / 16;
  __shared__ float mg_m[NWV][16], mg_l[NWV][16];
  __shared__ float mg_o[NWV][DBLK][64][4];
  [[maybe_unused]] __shared__ float rope_cs[ROPE ? D / 2 : 1], rope_sn[ROPE ? D / 2 : 1];

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

  const bool row_valid = r16 < rows;
  const int tok = row0 + (row_valid ? r16 / G : 0);
  const int head = gkv * G + (row_valid ? r16 % G : 0);
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  bf16x8_t qf[KSTEPS];
  [[maybe_unused]] bf16x8_t knew[KSTEPS];     // ROPE: the token's key, as this lane's fragments
  [[maybe_unused]] bf16_t vnew[DBLK];         // and its value at head-dim elements db * 16 + r16
  [[maybe_unused]] float xq[KSTEPS][8], xk[KSTEPS][8];
  [[maybe_unused]] float wq[KSTEPS][8], wk[KSTEPS][8];
  [[maybe_unused]] float freq = 0.f;
  if constexpr (ROPE) {
    // the raw rows, the norms' weights and the frequencies are requested first of all: none
    // of them waits for anything, and the norm is done by the time the position has arrived
    const bf16_t* row = rope.qkv + (size_t)tok * (nh + 2 * nkv) * D;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      load8<bf16_t>(row + (size_t)head * D + ks * 32 + grp * 8, xq[ks]);
      load8<bf16_t>(row + (size_t)(nh + gkv) * D + ks * 32 + grp * 8, xk[ks]);
      if (rope.q_norm_w) load8<float>(rope.q_norm_w + ks * 32 + grp * 8, wq[ks]);
      if (rope.k_norm_w) load8<float>(rope.k_norm_w + ks * 32 + grp * 8, wk[ks]);
    }
#pragma unroll
    for (int db = 0; db < DBLK; ++db) vnew[db] = row[(size_t)(nh + nkv + gkv) * D + db * 16 + r16];
    freq = rope.inv_freq[tid & (D / 2 - 1)];
  } else {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      qf[ks] = row_valid ? *reinterpret_cast<const bf16x8_t*>(
                               q + ((size_t)tok * nh + head) * D + ks * 32 + grp * 8)
                         : zero8;
  }

  f32x4_t o[DBLK];
#pragma unroll
  for (int db = 0; db < DBLK; ++db) o[db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // One tile's keys and values as first-operand fragments in registers; the next tile
  // is fetched while this one is being computed.
  //
  // Which key sits in which row of a 16-row block is free as long as scores, masks
  // and values agree.  Rows are dealt so that a lane's scores of blocks 2kk and
  // 2kk + 1 are those of EIGHT consecutive keys: row r of block jb is key
  //   (jb / 2) * 32 + (r / 4) * 8 + (jb % 2) * 4 + r % 4          of the tile,
  // so lane group grp ends up with keys kk * 32 + grp * 8 .. + 7, in that order, as
  // the 8 k-slots of the second product.  The values of those eight keys for one
  // head-dim element lie side by side in the page: vf[db][kk] is ONE 16-byte load
  // (two of 8 bytes when the page size is no multiple of 8).
  bf16x8_t kf[4][KSTEPS];
  bf16x8_t vf[DBLK][2];
  // Block-table entries are read whether or not their keys turn out to be in range
  // (an entry beyond the table reads the last one, an unused entry, -1, page 0).
  const int last_entry = bt_stride - 1;
  const int ps_shift = page_shift_of(page_size);
  const bool wide = page_size % 8 == 0;
  const int krow_in_pair = (r16 >> 2) * 8 + (r16 & 3);   // + (jb / 2) * 32 + (jb % 2) * 4
  auto entry_of = [&](int key) {
    const int e = page_entry(key, page_size, ps_shift);
    return table[e < last_entry ? e : last_entry];
  };
  // With pages of 16, 32, 64 ... keys a block of 16 keys lies in one page (tiles start at
  // multiples of 16 keys): four entries a tile, the same for the whole wave.  The entries
  // of the wave's next sixteen tiles are read by ONE vector load, lane i * 4 + b taking
  // block b of the i-th tile, and handed out lane by lane: a tile's loads of keys and
  // values then wait for no table lookup of their own.
  int tbl = 0;
  auto load_entries = [&](int first_tile0) {
    const int key = first_tile0 + (lane >> 2) * (NWV * AM_KT) + (lane & 3) * 16;
    const int e = key >> (ps_shift >= 4 ? ps_shift : 4);
    tbl = table[e < last_entry ? e : last_entry];
  };
  // `nth`: which of the wave's tiles since the entries were read (0 .. 15)
  auto fetch = [&](int tile0, int nth, bf16x8_t (&kfr)[4][KSTEPS], bf16x8_t (&vfr)[DBLK][2]) {
    int kpage[4], vpage[4];      // vpage: per run of 4 keys, kk * 2 + half
    if (ps_shift >= 4) {
      const int first = __builtin_amdgcn_readfirstlane(nth) * 4;
      int pg[4];
#pragma unroll
      for (int b = 0; b < 4; ++b) pg[b] = __builtin_amdgcn_readlane(tbl, first + b);
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        kpage[jb] = (r16 & 8) ? pg[(jb >> 1) * 2 + 1] : pg[(jb >> 1) * 2];
        vpage[jb] = (grp & 2) ? pg[(jb >> 1) * 2 + 1] : pg[(jb >> 1) * 2];
      }
    } else {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        kpage[jb] = entry_of(tile0 + (jb >> 1) * 32 + (jb & 1) * 4 + krow_in_pair);
        vpage[jb] = entry_of(tile0 + (jb >> 1) * 32 + grp * 8 + (jb & 1) * 4);
      }
    }
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const int kp = tile0 + (jb >> 1) * 32 + (jb & 1) * 4 + krow_in_pair;
      const int page = kpage[jb] < 0 ? 0 : kpage[jb];
      const bf16_t* krow = kv + ((((size_t)page * 2) * nkv + gkv) * page_size +
                                 page_offset(kp, page_size, ps_shift)) * D;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        kfr[jb][ks] = *reinterpret_cast<const bf16x8_t*>(krow + ks * 32 + grp * 8);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int kp = tile0 + kk * 32 + grp * 8;          // this lane's eight keys
      const int page_a = vpage[2 * kk] < 0 ? 0 : vpage[2 * kk];
      const int page_b = vpage[2 * kk + 1] < 0 ? 0 : vpage[2 * kk + 1];
      const bf16_t* va = kv + (((size_t)page_a * 2 + 1) * nkv + gkv) * page_size * D +
                         page_offset(kp, page_size, ps_shift);
      const bf16_t* vb = kv + (((size_t)page_b * 2 + 1) * nkv + gkv) * page_size * D +
                         page_offset(kp + 4, page_size, ps_shift);
#pragma unroll
      for (int db = 0; db < DBLK; ++db) {
        const size_t row = (size_t)(db * 16 + r16) * page_size;
        bf16x8_t x;
        if (wide) {
          x = *reinterpret_cast<const bf16x8_t*>(va + row);
        } else {
          const bf16x4_t xa = *reinterpret_cast<const bf16x4_t*>(va + row);
          const bf16x4_t xb = *reinterpret_cast<const bf16x4_t*>(vb + row);
          x = __builtin_shufflevector(xa, xb, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        vfr[db][kk] = x;
      }
    }
  };

  // Without a window the wave's first tile is known before the positions have arrived
  // (a range starts where the launch says): its entries, keys and values are requested
  // at once, so that the kernel's start is two trips to memory (entries and positions
  // side by side, then keys and values) and not three.  A wave whose tile turns out to
  // lie beyond the context has loaded in vain (from inside the pool, as every load here).
  const bool early = window == 0;
  if (early) {
    const int first_tile0 = (nsplit == 1 ? 0 : z * keys_per_split) + wave * AM_KT;
    if (ps_shift >= 4) load_entries(first_tile0);
    fetch(first_tile0, 0, kf, vf);
  }

  const int pos_first = positions[row0];
  const int pos_last = positions[row0 + count - 1];
  const int pos_row = row_valid ? positions[tok] : -1;
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int hi = pos_last;
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;
  // (the token's own key and value are stored by whoever meets its position: ranges that
  // end before it would leave them out of the cache, so the last range takes what is left)
  if (ROPE && z == nsplit - 1) range_hi = hi;
  int tile_first = (lo / AM_KT) * AM_KT;
  if (tile_first < range_lo) tile_first = range_lo;

  int tile0 = tile_first + wave * AM_KT;
  if (!early && tile0 <= range_hi) {
    if (ps_shift >= 4) load_entries(tile0);
    fetch(tile0, 0, kf, vf);
  }
  if constexpr (ROPE) {
    // chunk ks * 4 + grp of a head is this lane's x[ks]; the sums of squares meet as in the
    // kernel this replaces: partners half the head apart first, then ever closer ones
    auto normalise = [&](float (&x)[KSTEPS][8], const float (&w)[KSTEPS][8]) {
      float ss[KSTEPS];
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) ss[ks] = rope_sum_squares8(x[ks]);
#pragma unroll
      for (int o = KSTEPS / 2; o > 0; o >>= 1)
#pragma unroll
        for (int ks = 0; ks < o; ++ks) ss[ks] += ss[ks + o];
      float t = ss[0];
      t += __shfl_xor(t, 32, ZA_WAVE);
      t += __shfl_xor(t, 16, ZA_WAVE);
      const float norm_scale = rope_rms_scale(t, D, rope.eps);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) rope_scale8(x[ks], norm_scale, w[ks]);
    };
    if (rope.q_norm_w) normalise(xq, wq);
    if (rope.k_norm_w) normalise(xk, wk);
    if (tid < D / 2) rope_angle(pos_last, freq, &rope_cs[tid], &rope_sn[tid]);
    __syncthreads();
    auto rotate = [&](float (&x)[KSTEPS][8], bf16x8_t (&frag)[KSTEPS]) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS / 2; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int p = ks * 32 + grp * 8 + i;
          const float cs = rope_cs[p], sn = rope_sn[p];
          const float lo = x[ks][i], hi = x[ks + KSTEPS / 2][i];
          x[ks][i] = rope_rotate_low(lo, hi, cs, sn);
          x[ks + KSTEPS / 2][i] = rope_rotate_high(hi, lo, cs, sn);
        }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) frag[ks][i] = (bf16_t)x[ks][i];
    };
    rotate(xq, qf);
    if (!row_valid) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = zero8;
    }
    rotate(xk, knew);
  }
  int nth = 0;
  for (; tile0 <= range_hi; tile0 += NWV * AM_KT) {
    bf16x8_t kfn[4][KSTEPS];
    bf16x8_t vfn[DBLK][2];
    const int next = tile0 + NWV * AM_KT;
    if (next <= range_hi) {
      if (++nth == 16) {
        nth = 0;
        if (ps_shift >= 4) load_entries(next);
      }
      fetch(next, nth, kfn, vfn);
    }
    if constexpr (ROPE) {
      // the tile with the token's own position (one wave of one workgroup meets it): key
      // and value are not in the cache yet, they go into the fragments here and from here
      // into the cache
      const int own = pos_last - tile0;
      if (own >= 0 && own < AM_KT) {
#pragma unroll
        for (int jb = 0; jb < 4; ++jb)
          if ((jb >> 1) * 32 + (jb & 1) * 4 + krow_in_pair == own) {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) kf[jb][ks] = knew[ks];
          }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (kk * 32 + grp * 8 + e == own) {
#pragma unroll
              for (int db = 0; db < DBLK; ++db) vf[db][kk][e] = vnew[db];
            }
        const int slot = rope.write_kv ? rope.slots[tok] : -1;
        if (slot >= 0) {
          const int page = slot / page_size, off = slot % page_size;
          if (r16 == 0) {
            bf16_t* dst = rope.kv_write + ((((size_t)page * 2) * nkv + gkv) * page_size + off) * D;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks)
              *reinterpret_cast<bf16x8_t*>(dst + ks * 32 + grp * 8) = knew[ks];
          }
          if (grp == 0) {
            bf16_t* dst = rope.kv_write + (((size_t)page * 2 + 1) * nkv + gkv) * page_size * D + off;
#pragma unroll
            for (int db = 0; db < DBLK; ++db) dst[(size_t)(db * 16 + r16) * page_size] = vnew[db];
          }
        }
      }
    }
    // A key that must not count is masked in the scores, whatever its row holds; its
    // values are cleared, since 0 * (not a number) would not be 0.  (Keys whose page is
    // not there, entry -1, lie outside [lo, range_hi] too.)
    if (tile0 < lo || tile0 + AM_KT - 1 > range_hi) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int kp = tile0 + kk * 32 + grp * 8;
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (kp + e < lo || kp + e > range_hi) vf[db][kk][e] = (bf16_t)0.f;
      }
    }

    f32x4_t s[4];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      s[jb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        s[jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[jb][ks], qf[ks], s[jb], 0, 0, 0);
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kp = tile0 + (jb >> 1) * 32 + grp * 8 + (jb & 1) * 4 + i;
        bool valid = kp <= pos_row && kp >= lo && kp <= range_hi;
        if (window > 0 && kp <= pos_row - window) valid = false;
        const float v = valid ? s[jb][i] * scale_log2e : -INFINITY;
        s[jb][i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = quad_max(tmax);
    // the running maximum as a whole number on the base-2 scale: every rescaling factor
    // is an exact power of two (see paged_attention_mfma_kernel)
    const float m_new = fmaxf(m, ceilf(tmax));
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float alpha = m > -INFINITY ? ldexpf(1.0f, (int)(m - m_use)) : 1.0f;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb)
#pragma unroll
      for (int i = 0; i < 4; ++i) s[jb][i] = __builtin_amdgcn_exp2f(s[jb][i] - m_use);
    m = m_new;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
    // the probabilities rounded for the second product; the sum that normalises the result
    // is the sum of the rounded values, as in paged_attention_mfma_kernel
    bf16x8_t pf[2];
    float psum = 0.f;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pf[kk][i] = (bf16_t)s[2 * kk][i];
        pf[kk][4 + i] = (bf16_t)s[2 * kk + 1][i];
        psum += (float)pf[kk][i] + (float)pf[kk][4 + i];
      }
    psum = quad_sum(psum);
    l = l * alpha + psum;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][kk], pf[kk], o[db], 0, 0, 0);
    if (next <= range_hi) {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) kf[jb][ks] = kfn[jb][ks];
      }
#pragma unroll
      for (int db = 0; db < DBLK; ++db) {
        vf[db][0] = vfn[db][0];
        vf[db][1] = vfn[db][1];
      }
    }
  }

  // merge the waves' partial results
  if (grp == 0) { mg_m[wave][r16] = m; mg_l[wave][r16] = l; }
#pragma unroll
  for (int db = 0; db < DBLK; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) mg_o[wave][db][lane][i] = o[db][i];
  __syncthreads();
  if (wave == 0 && row_valid) {
    float mx = mg_m[0][r16];
#pragma unroll
    for (int w = 1; w < NWV; ++w) mx = fmaxf(mx, mg_m[w][r16]);
    const float mu = mx > -INFINITY ? mx : 0.f;
    float wgt[NWV], total = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      wgt[w] = mg_m[w][r16] > -INFINITY ? ldexpf(1.0f, (int)(mg_m[w][r16] - mu)) : 0.f;
      total += mg_l[w][r16] * wgt[w];
    }
    const size_t orow = (size_t)tok * nh + head;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; ++w) acc = fmaf(mg_o[w][db][lane][i], wgt[w], acc);
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
                       part_ml, (float*)out, d, nsplit, 0);
  else
    hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), grid, block, 0, stream, part_acc,
                       part_ml, (bf16_t*)out, d, nsplit, 0);
  return za_launch_status();
}

template <int D, int KT>
static int launch_attention_mfma(const void* q, void* out, const void* kv, const int* block_table,
                                 int bt_stride, const int* positions, const int* wi_seq,
                                 const int* wi_row0, const int* wi_count, int n_items,
                                 int n_tokens, float* part_acc, float* part_ml, int nh, int nkv,
                                 int page_size, float scale, int window, int keys_per_split,
                                 int nsplit, hipStream_t stream) {
  constexpr int NW = 8, NS = AM_ROWS / (NW * 16);
  const size_t shmem = ((size_t)2 * KT * (D + 8) + (size_t)2 * D * (KT + 8)) * sizeof(bf16_t);
  auto kernel = paged_attention_mfma_kernel<D, NW, NS, KT>;
  static bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
    allowed = true;
  }
  if (n_items > 65535) return ZA_ERR_UNSUPPORTED;
  // the key/value head runs fastest, so that workgroups that follow each other (and
  // are dealt to the chip's eight dies in turn) read different heads' keys and values
  dim3 grid(nkv, n_items, nsplit), block(NW * 64);
  hipLaunchKernelGGL(kernel, grid, block, shmem, stream, (const bf16_t*)q, (bf16_t*)out,
                     (const bf16_t*)kv, block_table, bt_stride, positions, wi_seq, wi_row0,
                     wi_count, n_items, part_acc, part_ml, nh, nkv, page_size,
                     scale * 1.44269504088896341f, window, keys_per_split, nsplit);
  int rc = za_launch_status();
  if (rc != 0 || nsplit == 1) return rc;
  dim3 cgrid((unsigned)((size_t)n_tokens * nh)), cblock(64);
  hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), cgrid, cblock, 0, stream, part_acc,
                     part_ml, (bf16_t*)out, D, nsplit, 1);
  return za_launch_status();
}

// Matrix-core variant: bfloat16 only, head_dim 64 or 128, page sizes that are
// multiples of 4, a positive scale, work items of at most 128 / (nh / nkv) query
// tokens; contexts optionally cut as in za_paged_attention (partial results merged by
// the same combine kernel).  Returns ZA_ERR_UNSUPPORTED otherwise.
extern "C" int za_paged_attention_mfma(const void* q, void* out, const void* kv,
                                       const int* block_table, int bt_stride,
                                       const int* positions, const int* wi_seq,
                                       const int* wi_row0, const int* wi_count, int n_items,
                                       int n_tokens, float* part_acc, float* part_ml, int nh,
                                       int nkv, int d, int page_size, float scale, int window,
                                       int keys_per_split, int nsplit, int tile_keys,
                                       hipStream_t stream) {
  if (n_items == 0 || n_tokens == 0) return 0;
  if (nsplit < 1 || nsplit > 65535 ||
      (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0)))
    return ZA_ERR_ARG;
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || page_size <= 0 || bt_stride <= 0 ||
      !q || !out || !kv || !block_table || !positions || !wi_seq || !wi_row0 || !wi_count ||
      (tile_keys != 64 && tile_keys != 128))
    return ZA_ERR_ARG;
  const int G = nh / nkv;
  // (a page's elements, keys and values of all heads, must fit 32 bits: the kernel
  // multiplies page numbers by that stride in one instruction)
  if ((d != 64 && d != 128) || G > AM_ROWS || page_size % 4 != 0 || !(scale > 0.f) ||
      nkv > 65535 || 2ull * nkv * page_size * d > 0xffffffffull)
    return ZA_ERR_UNSUPPORTED;
#define ZA_AM_ARGS                                                                             \
  q, out, kv, block_table, bt_stride, positions, wi_seq, wi_row0, wi_count, n_items, n_tokens, \
      part_acc, part_ml, nh, nkv, page_size, scale, window, keys_per_split, nsplit, stream
  // tiles of 128 keys spread a tile's fixed work (running maximum, addresses) over twice
  // the scores: for long contexts; head size 128 keeps tiles of 64 (LDS)
  if (d == 64) return tile_keys == 128 ? launch_attention_mfma<64, 128>(ZA_AM_ARGS)
                                       : launch_attention_mfma<64, 64>(ZA_AM_ARGS);
  return launch_attention_mfma<128, 64>(ZA_AM_ARGS);
#undef ZA_AM_ARGS
}

template <bool ROPE>
static int launch_decode_mfma(const void* q, void* out, const void* kv, const int* block_table,
                              int bt_stride, const int* positions, const int* wi_seq,
                              const int* wi_row0, const int* wi_count, int n_items, int n_tokens,
                              float* part_acc, float* part_ml, int nh, int nkv, int d,
                              int page_size, float scale, int window, int keys_per_split,
                              int nsplit, const DecodeRope& rope, bool combine,
                              hipStream_t stream) {
  dim3 grid(n_items, nkv, nsplit), block(256);
  // Few workgroups (a small batch): eight waves each, so that a compute unit that
  // gets one workgroup still has eight waves' loads in flight.
  const long long workgroups = (long long)n_items * nkv * nsplit;
  if (d == 64 && workgroups <= ZA_DECODE_WIDE_BELOW) {
    hipLaunchKernelGGL((paged_attention_decode_mfma_kernel<64, 8, ROPE>), grid, dim3(512), 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, part_acc, part_ml, nh, nkv,
                       page_size, scale * 1.44269504088896341f, window, keys_per_split, nsplit, rope);
  } else if (d == 64) {
    hipLaunchKernelGGL((paged_attention_decode_mfma_kernel<64, 4, ROPE>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, part_acc, part_ml, nh, nkv,
                       page_size, scale * 1.44269504088896341f, window, keys_per_split, nsplit, rope);
  } else {
    hipLaunchKernelGGL((paged_attention_decode_mfma_kernel<128, 4, ROPE>), grid, block, 0, stream,
                       (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kv, block_table, bt_stride,
                       positions, wi_seq, wi_row0, wi_count, part_acc, part_ml, nh, nkv,
                       page_size, scale * 1.44269504088896341f, window, keys_per_split, nsplit, rope);
  }
  int rc = za_launch_status();
  if (rc != 0 || nsplit == 1 || !combine) return rc;
  dim3 cgrid((unsigned)((size_t)n_tokens * nh)), cblock(64);
  hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), cgrid, cblock, 0, stream, part_acc,
                     part_ml, (bf16_t*)out, d, nsplit, 1);
  return za_launch_status();
}

// The merge alone: `rows` (token, head) rows of bfloat16 `out` [rows][d] from the partial
// results of `nsplit` context ranges, maxima on the base-2 scale (the matrix-core kernels').
extern "C" int za_attention_combine(const float* part_acc, const float* part_ml, void* out,
                                    int rows, int d, int nsplit, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || d <= 0 || d > AT_MAX_D || nsplit < 1 || !part_acc || !part_ml || !out)
    return ZA_ERR_ARG;
  hipLaunchKernelGGL((attention_combine_kernel<bf16_t>), dim3((unsigned)rows), dim3(64), 0, stream,
                     part_acc, part_ml, (bf16_t*)out, d, nsplit, 1);
  return za_launch_status();
}

// Matrix-core decode variant: bfloat16, head_dim 64 or 128, page sizes that are
// multiples of 4, work items of at most 16 / (nh / nkv) query tokens, contexts
// optionally cut as in
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
  if ((d != 64 && d != 128) || G > 16 || page_size % 4 != 0 || nkv > 65535 || nsplit > 65535)
    return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  const DecodeRope none = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0};
  return launch_decode_mfma<false>(q, out, kv, block_table, bt_stride, positions, wi_seq, wi_row0,
                                   wi_count, n_items, n_tokens, part_acc, part_ml, nh, nkv, d,
                                   page_size, scale, window, keys_per_split, nsplit, none, true,
                                   stream);
}

// The same for a step in which every request brings one token, with the token's part of
// qk_norm_rope_kv_write in the kernel's prologue: `qkv` is the fused projection
// [n_tokens][nh + 2 nkv][d] as it leaves the product; queries and key get their per-head
// RMSNorm (weights may be null) and the rotation over the whole head with half pairing
// (rotary_dim == d, pairs (p, p + d / 2)), key and value go to the cache at `slots`
// (page * page_size + offset, -1: not stored).  The result and the cache hold the bits that
// za_qk_norm_rope_kv_write followed by za_paged_attention_decode_mfma leave.  With
// nsplit > 1 and `combine` 0 the partial results stay as they are in part_acc / part_ml
// (`out` is not written and may be null): whoever reads them merges them
// (za_attention_combine, or za_gemm_bf16_rows16_merged on its way in).
extern "C" int za_paged_attention_decode_mfma_rope(
    const void* qkv, void* out, void* kv, const int* block_table, int bt_stride,
    const int* positions, const int* slots, const float* q_norm_w, const float* k_norm_w,
    const float* inv_freq, float eps, int n_tokens, float* part_acc, float* part_ml, int nh,
    int nkv, int d, int page_size, float scale, int window, int keys_per_split, int nsplit,
    int combine, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || page_size <= 0 || bt_stride <= 0 ||
      nsplit < 1 || !qkv || !kv || !block_table || !positions || !slots || !inv_freq ||
      (!out && (combine || nsplit == 1)))
    return ZA_ERR_ARG;
  const int G = nh / nkv;
  if ((d != 64 && d != 128) || G > 16 || page_size % 4 != 0 || nkv > 65535 || nsplit > 65535)
    return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  const DecodeRope rope = {(const bf16_t*)qkv, slots, q_norm_w, k_norm_w, inv_freq, (bf16_t*)kv,
                           eps, 1};
  return launch_decode_mfma<true>(nullptr, out, kv, block_table, bt_stride, positions, nullptr,
                                  nullptr, nullptr, n_tokens, n_tokens, part_acc, part_ml, nh, nkv,
                                  d, page_size, scale, window, keys_per_split, nsplit, rope,
                                  combine != 0, stream);
}
