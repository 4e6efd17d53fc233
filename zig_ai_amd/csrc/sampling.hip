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

#include "common.h"

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

__global__ void __launch_bounds__(SM_THREADS)
sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const float* __restrict__ uniform, int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ float wave_tot[SM_THREADS / 64];
  __shared__ int found;
  __shared__ int last_kept;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (size_t)r * vocab;
  const float temp = temperature[r];
  const int chunk = (vocab + SM_THREADS - 1) / SM_THREADS;
  const int begin = tid * chunk < vocab ? tid * chunk : vocab;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;

  if (!(temp > 0.f)) {  // greedy: first index of the maximum
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin; i < end; ++i)
      if (row[i] > bv) { bv = row[i]; bi = i; }
    const float mx = block_max(bv, scratch);
    if (tid == 0) found = 0x7fffffff;
    __syncthreads();
    if (bv == mx && bi != 0x7fffffff) atomicMin(&found, bi);
    __syncthreads();
    if (tid == 0) out[r] = found == 0x7fffffff ? 0 : found;
    return;
  }

  const float inv_t = 1.0f / temp;
  float mx = -INFINITY;
  for (int i = begin; i < end; ++i) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, scratch);

  // top-k: the largest key with at least k values at or above it
  unsigned floor_key = 0u;
  const int k = top_k[r];
  if (k > 0 && k < vocab) {
    unsigned key = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = key | (1u << bit);
      float cnt = 0.f;
      for (int i = begin; i < end; ++i) cnt += ordered_key(row[i] * inv_t) >= cand ? 1.f : 0.f;
      cnt = block_sum(cnt, scratch);
      if (cnt >= (float)k) key = cand;
    }
    floor_key = key;
  }

  // top-p: the largest key whose values at or above it carry at least p of the mass
  const float p = top_p[r];
  if (p < 1.0f) {
    float mass = 0.f;
    for (int i = begin; i < end; ++i) {
      const float v = row[i] * inv_t;
      if (ordered_key(v) >= floor_key) mass += expf(v - mx);
    }
    mass = block_sum(mass, scratch);
    const float need = p * mass;
    unsigned key = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned cand = key | (1u << bit);
      float part = 0.f;
      for (int i = begin; i < end; ++i) {
        const float v = row[i] * inv_t;
        const unsigned kk = ordered_key(v);
        if (kk >= cand && kk >= floor_key) part += expf(v - mx);
      }
      part = block_sum(part, scratch);
      if (part >= need) key = cand;
    }
    if (key > floor_key) floor_key = key;
  }

  // the draw, in index order over the kept values
  float mine = 0.f;
  int my_last = -1;
  for (int i = begin; i < end; ++i) {
    const float v = row[i] * inv_t;
    if (ordered_key(v) >= floor_key) {
      const float e = expf(v - mx);
      mine += e;
      if (e > 0.f) my_last = i;
    }
  }
  // exclusive prefix of `mine` over the threads: scan inside each wave, then over waves
  const int lane = tid & 63, wave = tid >> 6;
  float incl = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_tot[wave] = incl;
  if (tid == 0) { found = 0x7fffffff; last_kept = -1; }
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < SM_THREADS / 64; ++w) {
    if (w < wave) before += wave_tot[w];
    total += wave_tot[w];
  }
  float acc = before + incl - mine;
  const float target = uniform[r] * total;
  if (my_last >= 0) atomicMax(&last_kept, my_last);
  for (int i = begin; i < end; ++i) {
    const float v = row[i] * inv_t;
    if (ordered_key(v) >= floor_key) {
      const float e = expf(v - mx);
      acc += e;
      if (e > 0.f && target <= acc) {
        atomicMin(&found, i);
        break;
      }
    }
  }
  __syncthreads();
  if (tid == 0) out[r] = found != 0x7fffffff ? found : (last_kept >= 0 ? last_kept : 0);
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

extern "C" int za_sample(const float* logits, int n_rows, int vocab, const float* temperature,
                         const int* top_k, const float* top_p, const float* uniform, int* out,
                         hipStream_t stream) {
  if (n_rows == 0) return 0;
  if (n_rows < 0 || vocab <= 0 || !logits || !temperature || !top_k || !top_p || !uniform || !out)
    return ZA_ERR_ARG;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SM_THREADS), 0, stream, logits, vocab,
                     temperature, top_k, top_p, uniform, out);
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
