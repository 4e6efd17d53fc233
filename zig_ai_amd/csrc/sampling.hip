// Choosing the next token from 32-bit logits on the device, one workgroup per row.
//
// Order of the steps as in the reference's sampler
// (/root/reference/src/transformer/pipeline.zig:25-150): repetition penalty, then
// temperature, then top-k, then top-p, then a draw.
//   * temperature <= 0: the first index of the maximum (pipeline.zig:30-32, 155-181);
//   * otherwise v = logit / temperature; top-k keeps v >= the k-th largest value
//     (pipeline.zig:80-99); top-p keeps the smallest set of largest values whose
//     probability reaches p (pipeline.zig:102-142; values equal to the last kept one
//     are all kept here); the draw returns the first kept index i, in index order,
//     with  sum_{j<=i} exp(v_j - max) >= u * sum_all  (pipeline.zig:39-52), u being
//     the row's uniform number in [0, 1) supplied by the host.
//   * the repetition penalty divides positive and multiplies negative logits of
//     listed tokens by the factor given for each (pipeline.zig:61-68).
#include <math.h>
#include <stdint.h>
#include <stdio.h>

#include <mutex>

#include "common.h"
#include "no_alloc.h"

#define SM_THREADS 1024

__device__ __forceinline__ unsigned ordered_key(float v) {
  const unsigned b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__global__ void __launch_bounds__(SM_THREADS)
argmax_kernel(const float* __restrict__ logits, int vocab, int* __restrict__ out) {
  __shared__ float best_v[SM_THREADS / 64];
  __shared__ int best_i[SM_THREADS / 64];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += SM_THREADS) {
    const float v = row[i];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SM_THREADS / 64; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

// Greedy choice for few rows of a large vocabulary: the row is cut into
// gridDim.y chunks so that more than a handful of workgroups read it; each
// writes its (maximum, first index) and `argmax_merge_kernel` picks the winner,
// the lower index among equal maxima.
__global__ void __launch_bounds__(SM_THREADS)
argmax_chunk_kernel(const float* __restrict__ logits, int vocab, float* __restrict__ part_v,
                    int* __restrict__ part_i) {
  __shared__ float best_v[SM_THREADS / 64];
  __shared__ int best_i[SM_THREADS / 64];
  const int chunk = (vocab + gridDim.y - 1) / gridDim.y;
  const int begin = blockIdx.y * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  const float* row = logits + (size_t)blockIdx.x * vocab;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += SM_THREADS) {
    const float v = row[i];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SM_THREADS / 64; ++w)
      if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
    part_v[blockIdx.x * gridDim.y + blockIdx.y] = bv;
    part_i[blockIdx.x * gridDim.y + blockIdx.y] = bi;
  }
}

__global__ void __launch_bounds__(64)
argmax_merge_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int chunks,
                    int* __restrict__ out) {
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const float v = part_v[blockIdx.x * chunks + c];
    const int i = part_i[blockIdx.x * chunks + c];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// ------------------------------------------------------------------ sampling
// One workgroup per row.  Thread t reads elements (j * 1024 + t) * VEC .. + VEC - 1
// of tile j: neighbouring lanes read neighbouring addresses, and index order is
// tile, then thread, then element.
//
// Thresholds.  top-k and top-p both ask for a key (ordered_key of v = logit / T)
// such that everything at or above it is kept.  Values are first counted into
// SM_BINS bins of mx - v (1/16 wide, the last bin takes the rest): count and
// probability mass per bin, then prefix sums over the bins name the bin in which
// a threshold lies, and only that bin's values (a list in LDS) are searched
// bit by bit, by one wave.  If a bin holds more values than the list (ties by the
// thousand, a flat row), the same search runs over the whole row instead, 32
// passes.  Masses are summed as 64-bit integers (exp(v - mx) in units of 2^-40):
// such sums do not depend on their order, so both searches find the same key,
// and the same key in every run.
#define SM_BINS 1024
#define SM_BIN_SCALE 16.0f
#define SM_LIST_MAX 4096
#define SM_MAX_TILES 256
#define SM_MASS_ONE 1099511627776.0f   // 2^40
static_assert(SM_BINS == SM_THREADS, "one bin per thread in the prefix sums");

typedef unsigned long long u64_t;

__device__ __forceinline__ float key_value(unsigned key) {
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}
__device__ __forceinline__ u64_t mass_units(float v, float mx) {
  return (u64_t)(__expf(v - mx) * SM_MASS_ONE);
}
// v <= mx.  Larger values land in lower bins; infinities and NaN in the last.
__device__ __forceinline__ int bin_of(float v, float mx) {
  return (int)fminf((mx - v) * SM_BIN_SCALE, (float)(SM_BINS - 1));
}
__device__ __forceinline__ u64_t shfl_xor_u64(u64_t v, int o) {
  const unsigned lo = __shfl_xor((unsigned)v, o, 64), hi = __shfl_xor((unsigned)(v >> 32), o, 64);
  return ((u64_t)hi << 32) | lo;
}
__device__ __forceinline__ u64_t shfl_up_u64(u64_t v, int o) {
  const unsigned lo = __shfl_up((unsigned)v, o, 64), hi = __shfl_up((unsigned)(v >> 32), o, 64);
  return ((u64_t)hi << 32) | lo;
}
__device__ __forceinline__ u64_t wave_sum_u64(u64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += shfl_xor_u64(v, o);
  return v;
}
// Sum over the workgroup, returned to every thread.
__device__ __forceinline__ u64_t block_sum_u64(u64_t v, u64_t* scratch) {
  v = wave_sum_u64(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  u64_t t = 0;
  for (int w = 0; w < SM_THREADS / 64; ++w) t += scratch[w];
  return t;
}

// VEC values from `base` on (in range as a whole: the vocabulary is a multiple of VEC).
template <int VEC>
__device__ __forceinline__ void load_values(const float* __restrict__ row, int base, float inv_t,
                                            float v[VEC]) {
  if (VEC == 4) {
    const float4 x = *reinterpret_cast<const float4*>(row + base);
    v[0] = x.x * inv_t; v[1] = x.y * inv_t; v[2] = x.z * inv_t; v[3] = x.w * inv_t;
  } else {
    v[0] = row[base] * inv_t;
  }
}

// f(index, value) for every value of the row this thread reads, in index order.
// The loads of SM_UNROLL tiles are issued before the first value is used: a row
// is read by one workgroup, which nothing else keeps busy while a load is under way.
#define SM_UNROLL 8
template <int VEC, typename F>
__device__ __forceinline__ void for_each_value(const float* __restrict__ row, int vocab,
                                               float inv_t, F f) {
  constexpr int STRIDE = SM_THREADS * VEC;
  int base = threadIdx.x * VEC;
  for (; base + (SM_UNROLL - 1) * STRIDE < vocab; base += SM_UNROLL * STRIDE) {
    float v[SM_UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < SM_UNROLL; ++u) load_values<VEC>(row, base + u * STRIDE, inv_t, v[u]);
#pragma unroll
    for (int u = 0; u < SM_UNROLL; ++u)
#pragma unroll
      for (int q = 0; q < VEC; ++q) f(base + u * STRIDE + q, v[u][q]);
  }
  for (; base < vocab; base += STRIDE) {
    float v[VEC];
    load_values<VEC>(row, base, inv_t, v);
#pragma unroll
    for (int q = 0; q < VEC; ++q) f(base + q, v[q]);
  }
}

// By one wave, over `n` keys in LDS: the largest key with at least `need` keys at
// or above it.
__device__ __forceinline__ unsigned wave_select_count(const unsigned* list, int n, int need) {
  const int lane = threadIdx.x & 63;
  unsigned key = 0u;
  for (int bit = 31; bit >= 0; --bit) {
    const unsigned cand = key | (1u << bit);
    int c = 0;
    for (int i0 = 0; i0 < n; i0 += 64) {
      const int i = i0 + lane;
      c += __popcll(__ballot(i < n && list[i] >= cand));
    }
    if (c >= need) key = cand;
  }
  return key;
}
// Mass of the keys at or above `floor_key`, plus `base`.
__device__ __forceinline__ u64_t wave_mass_ge(const unsigned* list, int n, unsigned floor_key,
                                             float mx) {
  const int lane = threadIdx.x & 63;
  u64_t s = 0;
  for (int i0 = 0; i0 < n; i0 += 64) {
    const int i = i0 + lane;
    if (i < n && list[i] >= floor_key) s += mass_units(key_value(list[i]), mx);
  }
  return wave_sum_u64(s);
}
// The largest key such that `base` plus the mass of the keys at or above it (and at
// or above `floor_key`) reaches `need`.
__device__ __forceinline__ unsigned wave_select_mass(const unsigned* list, int n, u64_t base,
                                                     u64_t need, unsigned floor_key, float mx) {
  const int lane = threadIdx.x & 63;
  unsigned key = 0u;
  for (int bit = 31; bit >= 0; --bit) {
    const unsigned cand = key | (1u << bit);
    u64_t s = 0;
    for (int i0 = 0; i0 < n; i0 += 64) {
      const int i = i0 + lane;
      if (i < n && list[i] >= cand && list[i] >= floor_key)
        s += mass_units(key_value(list[i]), mx);
    }
    if (base + wave_sum_u64(s) >= need) key = cand;
  }
  return key;
}

template <int VEC>
__global__ void __launch_bounds__(SM_THREADS)
sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const float* __restrict__ uniform, int* __restrict__ out, int whole_row_only) {
  __shared__ float scratch[16];
  __shared__ u64_t scratch64[16];
  __shared__ int cnt[2][SM_BINS];      // two copies (by lane parity) while counting; then
  __shared__ u64_t mass[2][SM_BINS];   // [0] = inclusive prefix sums, cnt[1] = the bin's count
  __shared__ unsigned list[SM_LIST_MAX];
  __shared__ int sh_i[8];
  __shared__ u64_t sh_q[2];
  __shared__ unsigned sh_u[2];
  __shared__ float sh_f[2];
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperature[r];

  if (!(temp > 0.f)) {  // greedy: first index of the maximum
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_each_value<VEC>(row, vocab, 1.0f, [&](int i, float v) {
      if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
    });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { scratch[wave] = bv; cnt[0][wave] = bi; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < SM_THREADS / 64; ++w)
        if (scratch[w] > bv || (scratch[w] == bv && cnt[0][w] < bi)) { bv = scratch[w]; bi = cnt[0][w]; }
      out[r] = bi == 0x7fffffff ? 0 : bi;
    }
    return;
  }

  const float inv_t = 1.0f / temp;
  float mx = -INFINITY;
  for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) { mx = fmaxf(mx, v); });
  mx = block_max(mx, scratch);

  // ---- the threshold: everything with ordered_key(v) >= floor_key is kept
  unsigned floor_key = 0u;
  const int k = top_k[r];
  const float p = top_p[r];
  const bool use_k = k > 0 && k < vocab, use_p = p < 1.0f;

  // searches over the whole row, for bins too full for the list
  auto row_select_count = [&](int need) {
    unsigned key = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = key | (1u << bit);
      u64_t c = 0;
      for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) { c += ordered_key(v) >= cand; });
      if (block_sum_u64(c, scratch64) >= (u64_t)need) key = cand;
    }
    return key;
  };
  auto row_mass_ge = [&](unsigned fl) {
    u64_t s = 0;
    for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) {
      if (ordered_key(v) >= fl) s += mass_units(v, mx);
    });
    return block_sum_u64(s, scratch64);
  };
  auto row_select_mass = [&](u64_t need, unsigned fl) {
    unsigned key = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = key | (1u << bit);
      u64_t s = 0;
      for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) {
        const unsigned kk = ordered_key(v);
        if (kk >= cand && kk >= fl) s += mass_units(v, mx);
      });
      if (block_sum_u64(s, scratch64) >= need) key = cand;
    }
    return key;
  };
  // the keys of one bin into `list` (the caller has checked that they fit)
  auto gather = [&](int bin) {
    if (tid == 0) sh_i[4] = 0;
    __syncthreads();
    for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) {
      if (bin_of(v, mx) == bin) {
        const int pos = atomicAdd(&sh_i[4], 1);
        if (pos < SM_LIST_MAX) list[pos] = ordered_key(v);
      }
    });
    __syncthreads();
  };

  if (use_k || use_p) {
    for (int b = tid; b < 2 * SM_BINS; b += SM_THREADS) {
      (&cnt[0][0])[b] = 0;
      (&mass[0][0])[b] = 0;
    }
    __syncthreads();
    const int copy = tid & 1;
    for_each_value<VEC>(row, vocab, inv_t, [&](int, float v) {
      const int b = bin_of(v, mx);
      atomicAdd(&cnt[copy][b], 1);
      atomicAdd(&mass[copy][b], mass_units(v, mx));
    });
    __syncthreads();
    // inclusive prefix sums over the bins, bin `tid` in this thread
    const int c = cnt[0][tid] + cnt[1][tid];
    const u64_t m = mass[0][tid] + mass[1][tid];
    int ci = c;
    u64_t mi = m;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int uc = __shfl_up(ci, o, 64);
      const u64_t um = shfl_up_u64(mi, o);
      if (lane >= o) { ci += uc; mi += um; }
    }
    if (lane == 63) { list[wave] = (unsigned)ci; scratch64[wave] = mi; }
    __syncthreads();
    for (int w = 0; w < wave; ++w) { ci += (int)list[w]; mi += scratch64[w]; }
    __syncthreads();
    cnt[0][tid] = ci;
    cnt[1][tid] = c;
    mass[0][tid] = mi;
    if (tid == 0) { sh_i[2] = -1; }
    __syncthreads();

    unsigned tau_k = 0u;
    u64_t mass_k = mass[0][SM_BINS - 1];
    int bk = SM_BINS;            // the bin of the k-th largest value
    bool list_holds_bk = false;
    if (use_k) {
      if (ci >= k && ci - c < k) { sh_i[0] = tid; sh_i[1] = ci - c; }   // one thread: vocab > k
      __syncthreads();
      bk = sh_i[0];
      const int above = sh_i[1], in_bin = cnt[1][bk];
      if (in_bin <= SM_LIST_MAX && !whole_row_only) {
        gather(bk);
        if (wave == 0) {
          const unsigned t = wave_select_count(list, in_bin, k - above);
          const u64_t mq = wave_mass_ge(list, in_bin, t, mx);
          if (lane == 0) { sh_u[0] = t; sh_q[0] = (bk > 0 ? mass[0][bk - 1] : 0) + mq; }
        }
        __syncthreads();
        tau_k = sh_u[0];
        mass_k = sh_q[0];
        list_holds_bk = true;
      } else {
        tau_k = row_select_count(k);
        mass_k = row_mass_ge(tau_k);
      }
    }
    unsigned tau_p = 0u;
    if (use_p) {
      u64_t need = p > 0.f ? (u64_t)((double)p * (double)mass_k) : 0;
      if (need == 0) need = 1;   // the largest value is always kept
      // the bin, above the top-k bin, in which the kept mass reaches `need`
      if (tid < bk && mi >= need && mi - m < need) sh_i[2] = tid;
      __syncthreads();
      const int bp = sh_i[2];
      if (bp >= 0) {
        const int in_bin = cnt[1][bp];
        const u64_t base = bp > 0 ? mass[0][bp - 1] : 0;
        if (in_bin <= SM_LIST_MAX && !whole_row_only) {
          gather(bp);
          if (wave == 0) {
            const unsigned t = wave_select_mass(list, in_bin, base, need, 0u, mx);
            if (lane == 0) sh_u[1] = t;
          }
          __syncthreads();
          tau_p = sh_u[1];
        } else {
          tau_p = row_select_mass(need, tau_k);
        }
      } else if (list_holds_bk) {   // inside the top-k bin, whose keys the list still holds
        if (wave == 0) {
          const unsigned t = wave_select_mass(list, cnt[1][bk], bk > 0 ? mass[0][bk - 1] : 0,
                                              need, tau_k, mx);
          if (lane == 0) sh_u[1] = t;
        }
        __syncthreads();
        tau_p = sh_u[1];
      } else {
        tau_p = row_select_mass(need, tau_k);
      }
    }
    floor_key = tau_k > tau_p ? tau_k : tau_p;
    __syncthreads();   // the bins are done with: their memory now holds the segment sums
  }

  // ---- the draw, in index order over the kept values.  A segment is what one wave
  // reads of one tile (64 * VEC consecutive values); segments in index order are
  // tile-major, wave-minor.
  float* seg = reinterpret_cast<float*>(&mass[0][0]);   // SM_MAX_TILES * 16 sums
  const int n_tiles = (vocab + SM_THREADS * VEC - 1) / (SM_THREADS * VEC);
  const int n_seg = n_tiles * (SM_THREADS / 64);
  for (int j0 = 0; j0 < n_tiles; j0 += SM_UNROLL) {
    float v[SM_UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < SM_UNROLL; ++u) {
      const int base = ((j0 + u) * SM_THREADS + tid) * VEC;
      if (base < vocab) load_values<VEC>(row, base, inv_t, v[u]);
    }
#pragma unroll
    for (int u = 0; u < SM_UNROLL; ++u) {
      const int base = ((j0 + u) * SM_THREADS + tid) * VEC;
      float e = 0.f;
      if (base < vocab) {
#pragma unroll
        for (int q = 0; q < VEC; ++q)
          if (ordered_key(v[u][q]) >= floor_key) e += __expf(v[u][q] - mx);
      }
      e = wave_sum(e);
      if (lane == 0 && j0 + u < n_tiles) seg[(j0 + u) * (SM_THREADS / 64) + wave] = e;
    }
  }
  if (tid == 0) { sh_i[5] = 0x7fffffff; sh_i[6] = -1; }
  __syncthreads();
  // prefix sums over the segments: a run of consecutive segments per thread
  const int per = (n_seg + SM_THREADS - 1) / SM_THREADS;
  const int s0 = tid * per < n_seg ? tid * per : n_seg;
  const int s1 = s0 + per < n_seg ? s0 + per : n_seg;
  float mine = 0.f;
  for (int sgm = s0; sgm < s1; ++sgm) mine += seg[sgm];
  float incl = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < SM_THREADS / 64; ++w) {
    if (w < wave) before += scratch[w];
    total += scratch[w];
  }
  const float target = uniform[r] * total;
  {
    float acc = before + incl - mine;
    for (int sgm = s0; sgm < s1; ++sgm) {
      const float w = seg[sgm];
      if (w > 0.f) {
        if (target <= acc + w) atomicMin(&sh_i[5], sgm);
        atomicMax(&sh_i[6], sgm);
      }
      acc += w;
    }
  }
  __syncthreads();
  const bool reached = sh_i[5] != 0x7fffffff;
  const int pick = reached ? sh_i[5] : sh_i[6];   // else: the last segment with any mass
  if (pick < 0) {                                  // nothing has mass (all -inf)
    if (tid == 0) out[r] = 0;
    return;
  }
  if (pick >= s0 && pick < s1) {                   // its owner knows what lies before it
    float acc = before + incl - mine;
    for (int sgm = s0; sgm < pick; ++sgm) acc += seg[sgm];
    sh_f[0] = acc;
  }
  __syncthreads();
  if (wave == pick % (SM_THREADS / 64)) {
    const int base = ((pick / (SM_THREADS / 64)) * SM_THREADS + tid) * VEC;
    float e[VEC];
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < VEC; ++q) e[q] = 0.f;
    if (base < vocab) {
      float v[VEC];
      load_values<VEC>(row, base, inv_t, v);
#pragma unroll
      for (int q = 0; q < VEC; ++q)
        if (ordered_key(v[q]) >= floor_key) e[q] = __expf(v[q] - mx);
    }
#pragma unroll
    for (int q = 0; q < VEC; ++q) sum += e[q];
    float li = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(li, o, 64);
      if (lane >= o) li += up;
    }
    float acc = sh_f[0] + li - sum;
    int first = 0x7fffffff, last = -1;
#pragma unroll
    for (int q = 0; q < VEC; ++q) {
      acc += e[q];
      if (e[q] > 0.f) {
        if (reached && target <= acc && first == 0x7fffffff) first = base + q;
        last = base + q;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const int of = __shfl_xor(first, o, 64), ol = __shfl_xor(last, o, 64);
      first = of < first ? of : first;
      last = ol > last ? ol : last;
    }
    if (lane == 0) out[r] = first != 0x7fffffff ? first : (last >= 0 ? last : 0);
  }
}

__global__ void __launch_bounds__(256)
repetition_penalty_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ rows,
                          const int* __restrict__ tokens, const float* __restrict__ factors,
                          int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const int tok = tokens[e];
  if (tok < 0 || tok >= vocab) return;
  float* p = logits + (size_t)rows[e] * vocab + tok;
  const float v = *p;
  if (v > 0.f) *p = v / factors[e];
  else if (v < 0.f) *p = v * factors[e];
}

// `part_v` / `part_i`: workspace of n_rows * chunks entries each when chunks > 1.
extern "C" int za_argmax(const float* logits, int n_rows, int vocab, int* out, float* part_v,
                         int* part_i, int chunks, hipStream_t stream) {
  if (n_rows == 0) return 0;
  if (n_rows < 0 || vocab <= 0 || !logits || !out || chunks < 1) return ZA_ERR_ARG;
  if (chunks == 1) {
    hipLaunchKernelGGL(argmax_kernel, dim3(n_rows), dim3(SM_THREADS), 0, stream, logits, vocab,
                       out);
    return za_launch_status();
  }
  if (!part_v || !part_i || chunks > 65535) return ZA_ERR_ARG;
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(n_rows, chunks), dim3(SM_THREADS), 0, stream,
                     logits, vocab, part_v, part_i);
  int rc = za_launch_status();
  if (rc != 0) return rc;
  hipLaunchKernelGGL(argmax_merge_kernel, dim3(n_rows), dim3(64), 0, stream, part_v, part_i,
                     chunks, out);
  return za_launch_status();
}

// ---------------------------------------------- greedy choice without allocation
// The workspace of the chunked argmax for callers that cannot allocate (no_alloc.h):
// ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS maxima (32-bit floats), then as many indices.  Host
// code never uses the array's name as an address (it is a stand-in there): the device
// address is asked for once per device and kept.
static __device__ __align__(256) unsigned char scratch[ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS * 8];

#define ZA_NO_ALLOC_MAX_DEVICES 64
static void* scratch_of_device[ZA_NO_ALLOC_MAX_DEVICES];     // null until asked for
static std::mutex scratch_lock;
static thread_local char no_alloc_error[192];

extern "C" const char* za_no_alloc_last_error(void) { return no_alloc_error; }

// The current device's copy of `scratch` into *out.  0, or the failed call's hipError_t
// (ZA_ERR_UNSUPPORTED for a device number beyond the table) with the reason in
// no_alloc_error.
static int scratch_address(void** out) {
  *out = nullptr;
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    snprintf(no_alloc_error, sizeof no_alloc_error, "za_argmax_no_alloc: hipGetDevice: %s",
             hipGetErrorString(e));
    return (int)e;
  }
  if (device < 0 || device >= ZA_NO_ALLOC_MAX_DEVICES) {
    snprintf(no_alloc_error, sizeof no_alloc_error,
             "za_argmax_no_alloc: device %d is beyond the %d this library keeps an address for",
             device, ZA_NO_ALLOC_MAX_DEVICES);
    return ZA_ERR_UNSUPPORTED;
  }
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (!scratch_of_device[device]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e == hipSuccess && !ptr) e = hipErrorInvalidSymbol;
    if (e != hipSuccess) {
      snprintf(no_alloc_error, sizeof no_alloc_error,
               "za_argmax_no_alloc: hipGetSymbolAddress on device %d: %s", device,
               hipGetErrorString(e));
      return (int)e;
    }
    scratch_of_device[device] = ptr;
  }
  *out = scratch_of_device[device];
  return 0;
}

extern "C" int za_argmax_no_alloc(const float* logits, int n_rows, int vocab, int* out,
                                  int chunks, hipStream_t stream) {
  no_alloc_error[0] = 0;
  if (n_rows == 0) return 0;
  if (n_rows < 0 || vocab <= 0 || !logits || !out || chunks < 1) {
    snprintf(no_alloc_error, sizeof no_alloc_error,
             "za_argmax_no_alloc: bad argument (n_rows %d, vocab %d, chunks %d, logits %p, out %p)",
             n_rows, vocab, chunks, (const void*)logits, (void*)out);
    return ZA_ERR_ARG;
  }
  if (chunks == 1) {                       // one workgroup a row: no partial results at all
    hipLaunchKernelGGL(argmax_kernel, dim3(n_rows), dim3(SM_THREADS), 0, stream, logits, vocab,
                       out);
    return za_launch_status();
  }
  if (chunks > 65535 || (long long)n_rows * chunks > ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS) {
    snprintf(no_alloc_error, sizeof no_alloc_error,
             "za_argmax_no_alloc: %d rows in %d chunks need %lld partial results, the array "
             "holds %d (and a row at most 65535 chunks)",
             n_rows, chunks, (long long)n_rows * chunks, ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS);
    return ZA_ERR_UNSUPPORTED;
  }
  void* base = nullptr;
  const int found = scratch_address(&base);
  if (found != 0) return found;
  float* part_v = reinterpret_cast<float*>(base);
  int* part_i = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(base) +
                                       (size_t)ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS * sizeof(float));
  // every entry the merge reads (n_rows * chunks of each) is written by the chunk kernel
  // of this call: what an earlier call left is never read
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(n_rows, chunks), dim3(SM_THREADS), 0, stream,
                     logits, vocab, part_v, part_i);
  int rc = za_launch_status();
  if (rc != 0) return rc;
  hipLaunchKernelGGL(argmax_merge_kernel, dim3(n_rows), dim3(64), 0, stream, part_v, part_i,
                     chunks, out);
  return za_launch_status();
}

// `whole_row_only`: search thresholds over the whole row only (the path for bins too
// full for the list; both paths find the same keys, which tests use).
extern "C" int za_sample(const float* logits, int n_rows, int vocab, const float* temperature,
                         const int* top_k, const float* top_p, const float* uniform, int* out,
                         int whole_row_only, hipStream_t stream) {
  if (n_rows == 0) return 0;
  if (n_rows < 0 || vocab <= 0 || !logits || !temperature || !top_k || !top_p || !uniform || !out)
    return ZA_ERR_ARG;
  const bool vec4 = vocab % 4 == 0 && ((uintptr_t)logits % 16) == 0;
  const int tiles = (vocab + SM_THREADS * (vec4 ? 4 : 1) - 1) / (SM_THREADS * (vec4 ? 4 : 1));
  if (tiles > SM_MAX_TILES) return ZA_ERR_UNSUPPORTED;   // a vocabulary beyond 1,048,576 (262,144)
  if (vec4)
    hipLaunchKernelGGL(sample_kernel<4>, dim3(n_rows), dim3(SM_THREADS), 0, stream, logits, vocab,
                       temperature, top_k, top_p, uniform, out, whole_row_only);
  else
    hipLaunchKernelGGL(sample_kernel<1>, dim3(n_rows), dim3(SM_THREADS), 0, stream, logits, vocab,
                       temperature, top_k, top_p, uniform, out, whole_row_only);
  return za_launch_status();
}

// Entries must name each (row, token) at most once; `factors[e]` is the penalty
// raised to the number of times the token occurred.
extern "C" int za_repetition_penalty(float* logits, int vocab, const int* rows, const int* tokens,
                                     const float* factors, int n, hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || vocab <= 0 || !logits || !rows || !tokens || !factors) return ZA_ERR_ARG;
  hipLaunchKernelGGL(repetition_penalty_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     logits, vocab, rows, tokens, factors, n);
  return za_launch_status();
}
