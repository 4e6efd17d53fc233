// Dense projections  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  with 32-bit
// accumulation.  Weights are row-major [out, in] as checkpoints store them (the
// layout the reference hands to its library GEMM:
// /root/reference/src/matmul/root.zig:292-313).
//
//   gemm_f32_kernel                 true 32-bit: LDS-tiled FMA, no matrix-core rounding modes
//   gemm_bf16_mfma_kernel           bfloat16 operands on the matrix cores (16x16x32), any M
//   gemm_bf16_skinny_kernel         bfloat16, M <= 64: streams W once, K split over the waves
//   gemm_bf16_rows16_kernel         bfloat16, M <= 16 (decoding): activations held in registers
//   gemm_bf16_rows16_swiglu_kernel  the same for the fused gate/up projection: writes
//                                   silu(gate) * up instead of the two products
//
// In every one of them an output element is a sum over k in an order that
// depends only on K, never on M or on the tile it falls in, so a token's result
// does not depend on which other tokens share the step (the bfloat16 kernels
// differ from each other in rounding only).
#include "common.h"

#include <mutex>
#include <type_traits>
#include <vector>

// ---------------------------------------------------------------- 32-bit FMA
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
gemm_f32_kernel(const TA* __restrict__ A, const float* __restrict__ W,
                const float* __restrict__ bias, TC* __restrict__ C, int M, int N, int K) {
  __shared__ float As[F32_BK][F32_BM + 4];
  __shared__ float Ws[F32_BK][F32_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int lrow = tid / 4;        // 0..63
  const int lk = (tid % 4) * 4;    // 0,4,8,12
  for (int k0 = 0; k0 < K; k0 += F32_BK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + j][lrow] = (am < M && k < K) ? to_f32<TA>(A[(size_t)am * K + k]) : 0.f;
      Ws[lk + j][lrow] = (wn < N && k < K) ? W[(size_t)wn * K + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F32_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      C[(size_t)m * N + n] = from_f32<TC>(v);
    }
  }
}

// ------------------------------------------------------- bfloat16, tiled MFMA
// Workgroup tile 128x128, K step 64; four waves in a 2x2 arrangement, each
// owning 64x64 = 4x4 matrix-core tiles of 16x16.  Operand layout of
// v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k (l / 16) * 8 .. + 7 of
// either operand and receives rows (l / 16) * 4 .. + 3, column (l % 16) of the product.
#define MF_BM 128
#define MF_BN 128
#define MF_BK 64
#define MF_LD (MF_BK + 8)  // padded row, in elements: spreads rows over LDS banks

template <typename TC>
__global__ void __launch_bounds__(256)
gemm_bf16_mfma_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                      const float* __restrict__ bias, TC* __restrict__ C, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16_t As[MF_BM * MF_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[MF_BN * MF_LD];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * MF_BM, n0 = blockIdx.x * MF_BN;

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // Each thread moves 4 + 4 vectors of 8 elements per K step.
  const int lrow = tid >> 3;        // 0..31, + 32 * i
  const int lcol = (tid & 7) * 8;   // element offset within the K step
  bf16x8_t ra[4], rw[4];
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = lrow + 32 * i;
      const int k = k0 + lcol;
      const int am = m0 + row, wn_ = n0 + row;
      ra[i] = (am < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(A + (size_t)am * K + k) : zero8;
      rw[i] = (wn_ < N && k < K) ? *reinterpret_cast<const bf16x8_t*>(W + (size_t)wn_ * K + k) : zero8;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = lrow + 32 * i;
      *reinterpret_cast<bf16x8_t*>(As + row * MF_LD + lcol) = ra[i];
      *reinterpret_cast<bf16x8_t*>(Ws + row * MF_LD + lcol) = rw[i];
    }
  };

  fetch(0);
  stash();
  __syncthreads();
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  for (int k0 = 0; k0 < K; k0 += MF_BK) {
    const bool more = k0 + MF_BK < K;
    if (more) fetch(k0 + MF_BK);
#pragma unroll
    for (int ks = 0; ks < MF_BK; ks += 32) {
      bf16x8_t fa[4], fw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fa[i] = *reinterpret_cast<const bf16x8_t*>(
            As + (wm * 64 + i * 16 + frag_row) * MF_LD + ks + frag_k);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        fw[j] = *reinterpret_cast<const bf16x8_t*>(
            Ws + (wn * 64 + j * 16 + frag_row) * MF_LD + ks + frag_k);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      stash();
      __syncthreads();
    }
  }

  const int out_col = lane & 15, out_row = (lane >> 4) * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn * 64 + j * 16 + out_col;
      if (n >= N) continue;
      const float b = bias ? bias[n] : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + wm * 64 + i * 16 + out_row + r;
        if (m < M) C[(size_t)m * N + n] = from_f32<TC>(acc[i][j][r] + b);
      }
    }
  }
}

// ---------------------------------------------------- bfloat16, few rows (decode)
// One workgroup per 16 output columns; its four waves take interleaved K chunks
// and their partial tiles are added in wave order through LDS.  W plays the
// first matrix-core operand (16 weight rows), the activations the second (16
// tokens), so a lane ends up with 4 consecutive output columns of one token.
#define SK_KSTEP 32
#define SK_UNROLL 4

template <int MT, typename TC>
__global__ void __launch_bounds__(256)
gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                        const float* __restrict__ bias, TC* __restrict__ C, int M, int N, int K) {
  __shared__ float red[4][MT][64][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 16;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int wrow = n0 + frag_row;
  const bool wvalid = wrow < N;
  const bf16_t* wp = W + (size_t)(wvalid ? wrow : 0) * K + frag_k;
  bool avalid[MT];
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + frag_row;
    avalid[t] = m < M;
    ap[t] = A + (size_t)(avalid[t] ? m : 0) * K + frag_k;
  }

  const int kstride = 4 * SK_KSTEP * SK_UNROLL;
  for (int kb = wave * SK_KSTEP * SK_UNROLL; kb < K; kb += kstride) {
    bf16x8_t fw[SK_UNROLL];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = kb + u * SK_KSTEP;
      fw[u] = (wvalid && k + frag_k < K) ? *reinterpret_cast<const bf16x8_t*>(wp + k) : zero8;
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = kb + u * SK_KSTEP;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8_t fa = (avalid[t] && k + frag_k < K)
                                ? *reinterpret_cast<const bf16x8_t*>(ap[t] + k) : zero8;
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[u], fa, acc[t], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][lane][r] = acc[t][r];
  __syncthreads();
  if (wave == 0) {
    const int m_in = lane & 15, nn = n0 + (lane >> 4) * 4;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + m_in;
      if (m >= M) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = nn + r;
        if (n >= N) continue;
        float v = red[0][t][lane][r] + red[1][t][lane][r];
        v += red[2][t][lane][r];
        v += red[3][t][lane][r];
        if (bias) v += bias[n];
        C[(size_t)m * N + n] = from_f32<TC>(v);
      }
    }
  }
}

// ------------------------------------------- bfloat16, at most 16 rows (decode)
// The activations of a decode step are few: every wave keeps its slice of them
// (16 tokens x KSTEPS * 32 elements of K) in registers for the whole kernel and
// streams weight rows past them, 16 rows at a time with all of a row group's
// loads in flight at once.  The NW waves of a workgroup split K; their partial
// tiles meet in LDS (double-buffered, one barrier per row group) and wave 0
// writes the sum.  A workgroup walks `groups_per_block` consecutive row groups.
//
// K may also be split over workgroups (gridDim.y ranges of NW * KSTEPS * 32): each
// range then writes a 32-bit partial result [range][M][N] that the consumer adds up
// (the bias goes into range 0).
//
// With `accumulate` the result is not stored but added to the 32-bit tensor C with
// floating-point atomics (C is then the residual stream, and the ranges of K meet
// there instead of in a stack): the order of these additions is the hardware's, so
// the sum is reproducible to rounding only.
// The activations of the decode kernels may also be a norm that has not run yet:
// rows of the 32-bit residual stream `x` (row m of the product is row rows[m] of
// the stream when `rows` is given) and an RMSNorm's weight and eps
// (/root/reference/src/transformer/norm.zig:6-33).  Every workgroup then reads the
// rows itself (they are few and come from L2) and a kernel between the producer of
// the stream and this product is saved.  The row's scale is a factor common to all of
// its elements, so it is applied to the 32-bit sums instead of to the operands:
//   y[m, n] = (1 / sqrt(mean_k(x[m, k]^2) + eps)) * sum_k W[n, k] * bf16(x[m, k] * weight[k])
// with the sum of squares in 32-bit from the unrounded x; the operands are rounded to
// bfloat16 once, as they are when the norm runs as a kernel of its own.  The
// workgroup's waves must cover all of K, and K must be a multiple of a wave's 512.
struct NormedRowsArg {
  const float* x;
  const int* rows;
  const float* weight;
  float eps;
};

// The scale of row m from the waves' sums of squares, added in a fixed order.
template <int NW>
__device__ __forceinline__ float normed_row_scale(const float (&ssw)[NW][16], int m, int K, float eps) {
  float total = ssw[0][m];
#pragma unroll
  for (int w = 1; w < NW; ++w) total += ssw[w][m];
  return 1.0f / sqrtf(total / (float)K + eps);
}

// The step's rows reach the waves through LDS (STAGED): a wave reads its slice of K of
// every row with one or two instructions a row, whole cache lines side by side, and takes
// the matrix-core fragments out of LDS.  Fragment loads straight from memory ask for every
// line of the rows twice (each instruction takes 64 bytes of 16 rows), and with hundreds of
// workgroups asking for the same few lines at a kernel's start that is what a step of
// few rows waits for: measured at 8 rows, gate|up of 8192 x 2048, 15.1 us with fragment
// loads, 14.3 staged, 13.4 with no rows at all.  A staged row of a wave's slice takes
// ROWS16_STAGE_STRIDE elements (eight more than the slice: the sixteen lanes that read
// one step of sixteen rows then fall into different banks).
#define ROWS16_STAGE_STRIDE (16 * 32 + 8)
#define ROWS16_STAGE_ROWS 8
extern __shared__ __attribute__((aligned(16))) unsigned char rows16_staged[];

// Nine to sixteen rows pass through the same eight places of LDS in two turns: the lanes
// whose fragment row lies in the first eight rows take their fragments, then the other
// eight rows are staged over them (a wave's LDS operations run in order).
__host__ __device__ inline int rows16_stage_places(int M) {
  return M < ROWS16_STAGE_ROWS ? M : ROWS16_STAGE_ROWS;
}
__host__ __device__ inline size_t rows16_stage_bytes(int nw, int M) {
  return (size_t)nw * rows16_stage_places(M) * ROWS16_STAGE_STRIDE * sizeof(bf16_t);
}

// The fragments of the wave's slice for the lanes whose row is one of rows r0 .. r0 + 7,
// out of the rows the wave staged itself (no barrier).  A lane without a row (row >= M)
// takes place 0 in the first turn.
template <int KSTEPS>
__device__ __forceinline__ void staged_fragments(bf16x8_t (&xa)[KSTEPS], const bf16_t* mine, int M,
                                                 int lane, int r0) {
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const bool valid = frag_row < M;
  if ((valid ? frag_row & 8 : 0) != r0) return;
  const bf16_t* fr = mine + (valid ? frag_row & 7 : 0) * ROWS16_STAGE_STRIDE + frag_k;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) xa[s] = *reinterpret_cast<const bf16x8_t*>(fr + s * 32);
}

// bfloat16 rows A [M, K], M <= 16; `kslice` is the first k of the wave's slice.  K is a
// multiple of 8, so a lane's eight elements are inside K or outside together; outside,
// zeros are staged (the address read is moved inside the operand).
template <int KSTEPS, typename Prefetch>
__device__ __forceinline__ void stage_rows(bf16x8_t (&xa)[KSTEPS], const bf16_t* __restrict__ A,
                                           int M, int K, int kslice, bf16_t* mine, int lane,
                                           Prefetch&& prefetch) {
  static_assert(KSTEPS == 16, "one instruction of a wave covers a row's slice of 512 elements");
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int k = kslice + lane * 8;
  const bool kin = k < K;
  const bf16_t* src = A + (kin ? k : 0);
  bf16x8_t v[2 * ROWS16_STAGE_ROWS];
#pragma unroll
  for (int r = 0; r < 2 * ROWS16_STAGE_ROWS; ++r)
    if (r < M) v[r] = *reinterpret_cast<const bf16x8_t*>(src + (size_t)r * K);
  // (weights requested behind the rows arrive while the rows pass through LDS)
  __builtin_amdgcn_sched_barrier(0);
  prefetch();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r0 = 0; r0 < 2 * ROWS16_STAGE_ROWS; r0 += ROWS16_STAGE_ROWS) {
    if (r0 > 0 && M <= r0) break;
#pragma unroll
    for (int r = 0; r < ROWS16_STAGE_ROWS; ++r)
      if (r0 + r < M)
        *reinterpret_cast<bf16x8_t*>(mine + r * ROWS16_STAGE_STRIDE + lane * 8) = kin ? v[r0 + r] : zero8;
    staged_fragments<KSTEPS>(xa, mine, M, lane, r0);
  }
}

// Rows that await their norm (NormedRowsArg): a lane reads four elements of each half of
// the wave's slice of every row, adds up their squares, and stages bf16(x * weight); eight
// rows at a time, up to MAX_ROWS (8 or 16); the sums of squares of the slice of row r go
// to ssw[wave][r].  `prefetch` is called once the first eight rows are requested, by the
// waves inside K only.  Ends with a barrier.  The lanes' sums of squares of eight rows meet in a butterfly that halves the rows a lane
// carries at each of its first three steps: ten exchanges instead of six a row, and the
// same tree of additions for every row wherever it stands.
template <int NW, int KSTEPS, int MAX_ROWS, typename Prefetch>
__device__ __forceinline__ void stage_normed_rows(bf16x8_t (&xa)[KSTEPS],
                                                  const float* __restrict__ x,
                                                  const int* __restrict__ rows,
                                                  const float* __restrict__ weight, int M, int K,
                                                  int tid, float (&ssw)[NW][16], bf16_t* staged,
                                                  Prefetch&& prefetch) {
  static_assert(KSTEPS == 16, "two instructions of a wave cover a row's slice of 512 elements");
  const int lane = tid & 63, wave = tid >> 6;
  const bool inside = (wave + 1) * (KSTEPS * 32) <= K;      // the same for a whole wave
  bf16_t* mine = staged + (size_t)wave * rows16_stage_places(M) * ROWS16_STAGE_STRIDE;
  if (inside) {
    const int kw = wave * (KSTEPS * 32) + lane * 4;
    const f32x4_t n0 = *reinterpret_cast<const f32x4_t*>(weight + kw);
    const f32x4_t n1 = *reinterpret_cast<const f32x4_t*>(weight + kw + 256);
#pragma unroll
    for (int r0 = 0; r0 < MAX_ROWS; r0 += ROWS16_STAGE_ROWS) {
      if (r0 > 0 && M <= r0) break;
      f32x4_t v[ROWS16_STAGE_ROWS][2];
#pragma unroll
      for (int r = 0; r < ROWS16_STAGE_ROWS; ++r)
        if (r0 + r < M) {
          const float* src = x + (rows ? (size_t)rows[r0 + r] : (size_t)(r0 + r)) * K + kw;
          v[r][0] = *reinterpret_cast<const f32x4_t*>(src);
          v[r][1] = *reinterpret_cast<const f32x4_t*>(src + 256);
        }
      if (r0 == 0) {
        // the first weights are requested behind the rows and arrive while the rows are
        // worked on (loads return in the order in which they were issued)
        __builtin_amdgcn_sched_barrier(0);
        prefetch();
        __builtin_amdgcn_sched_barrier(0);
      }
      float p[ROWS16_STAGE_ROWS];
#pragma unroll
      for (int r = 0; r < ROWS16_STAGE_ROWS; ++r) {
        p[r] = 0.f;
        if (r0 + r < M) {
          bf16x4_t lo, hi;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a = v[r][0][e], b = v[r][1][e];
            p[r] += a * a;
            p[r] += b * b;
            lo[e] = (bf16_t)(a * n0[e]);
            hi[e] = (bf16_t)(b * n1[e]);
          }
          bf16_t* dst = mine + r * ROWS16_STAGE_STRIDE + lane * 4;
          *reinterpret_cast<bf16x4_t*>(dst) = lo;
          *reinterpret_cast<bf16x4_t*>(dst + 256) = hi;
        }
      }
      // rows 4-7 go to the upper half of the lanes, then rows 2-3 and 6-7 to the lanes with
      // bit 4, then the odd rows to the lanes with bit 3; three plain steps finish the sums
      float q[4], t[2];
      const bool b5 = lane & 32, b4 = lane & 16, b3 = lane & 8;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        q[i] = (b5 ? p[i + 4] : p[i]) + __shfl_xor(b5 ? p[i] : p[i + 4], 32, ZA_WAVE);
#pragma unroll
      for (int i = 0; i < 2; ++i)
        t[i] = (b4 ? q[i + 2] : q[i]) + __shfl_xor(b4 ? q[i] : q[i + 2], 16, ZA_WAVE);
      float u = (b3 ? t[1] : t[0]) + __shfl_xor(b3 ? t[0] : t[1], 8, ZA_WAVE);
      u += __shfl_xor(u, 4, ZA_WAVE);
      u += __shfl_xor(u, 2, ZA_WAVE);
      u += __shfl_xor(u, 1, ZA_WAVE);
      const int row = (b5 ? 4 : 0) + (b4 ? 2 : 0) + (b3 ? 1 : 0);
      if ((lane & 7) == 0) ssw[wave][r0 + row] = u;
      staged_fragments<KSTEPS>(xa, mine, M, lane, r0);
    }
  } else {
    const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) xa[s] = zero8;
    if (lane < 16) ssw[wave][lane] = 0.f;
  }
  __syncthreads();
}

// Rows that are an attention's output while it still lies in the partial results of its
// context ranges (MergedRowsArg): for range z of row (token, head), an accumulator of `d`
// head-dim elements and (maximum on the base-2 scale, sum).  The product's kernel merges
// them on the way in, with the arithmetic of attention_combine_kernel in its order (the
// same bits), and a kernel between the attention and its output projection is saved.
// K = heads * d; up to 16 ranges, up to 8 rows.
struct MergedRowsArg {
  const float* acc;     // [rows][heads][nsplit][d]
  const float* ml;      // [rows][heads][nsplit][2]
  int nsplit;
  int d;
};

template <int KSTEPS, int Z, typename Prefetch>
__device__ __forceinline__ void stage_merged_rows(bf16x8_t (&xa)[KSTEPS], const MergedRowsArg& mg,
                                                  int M, int K, int kslice, bf16_t* mine, int lane,
                                                  Prefetch&& prefetch) {
  static_assert(KSTEPS == 16, "one lane takes eight elements of a row's slice of 512");
  constexpr int RB = 16 / Z;                 // rows whose partial results are in flight at once
  static_assert(Z == 2 || Z == 4 || Z == 8 || Z == 16, "ranges in flight");
  const int k = kslice + lane * 8;
  const int heads = K / mg.d, head = k / mg.d, dim = k % mg.d;
#pragma unroll
  for (int rb = 0; rb < ROWS16_STAGE_ROWS; rb += RB) {
    if (rb > 0 && M <= rb) break;
    float2 ml[RB][Z];
    f32x4_t pa[RB][Z][2];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int z = 0; z < Z; ++z)
        if (rb + r < M && z < mg.nsplit) {
          const size_t part = ((size_t)(rb + r) * heads + head) * mg.nsplit + z;
          ml[r][z] = *reinterpret_cast<const float2*>(mg.ml + part * 2);
          pa[r][z][0] = *reinterpret_cast<const f32x4_t*>(mg.acc + part * mg.d + dim);
          pa[r][z][1] = *reinterpret_cast<const f32x4_t*>(mg.acc + part * mg.d + dim + 4);
        }
    if (rb == 0) {
      __builtin_amdgcn_sched_barrier(0);
      prefetch();
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int r = 0; r < RB; ++r)
      if (rb + r < M) {
        float mx = -INFINITY;
#pragma unroll
        for (int z = 0; z < Z; ++z)
          if (z < mg.nsplit) mx = fmaxf(mx, ml[r][z].x);
        float total = 0.f, acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
        for (int z = 0; z < Z; ++z)
          if (z < mg.nsplit && ml[r][z].x > -INFINITY) {
            const float w = ldexpf(1.0f, (int)(ml[r][z].x - mx));
            total += ml[r][z].y * w;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(pa[r][z][e >> 2][e & 3], w, acc[e]);
          }
        const float inv = total > 0.f ? 1.0f / total : 0.f;
        bf16x8_t v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (bf16_t)(acc[e] * inv);
        *reinterpret_cast<bf16x8_t*>(mine + (rb + r) * ROWS16_STAGE_STRIDE + lane * 8) = v;
      }
  }
  staged_fragments<KSTEPS>(xa, mine, M, lane, 0);
}

template <int NW, int KSTEPS, typename TC, bool NORM, bool STAGED, bool ROLL, bool MERGED = false>
__global__ void __launch_bounds__(NW * 64, 2)
gemm_bf16_rows16_kernel(const bf16_t* __restrict__ A, NormedRowsArg normed,
                        const bf16_t* __restrict__ W, const float* __restrict__ bias,
                        TC* __restrict__ C, int M, int N, int K, int groups_per_block,
                        int accumulate, MergedRowsArg merged) {
  __shared__ float red[2][NW][64][4];
  __shared__ float ssw[NW][16];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const int kbase = (blockIdx.y * NW + wave) * KSTEPS * 32 + frag_k;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int HALF = KSTEPS > 16 ? 16 : KSTEPS;   // weight fragments in flight at once

  bf16x8_t xa[KSTEPS];
  // FAST (the norm in the kernel, or staged rows: K is then a multiple of a wave's slice):
  // a wave is all inside K or idle, and a row group's weights are loaded without conditions
  // (a lane beyond N reads row N - 1; its sums are never stored), the first group's while
  // the rows are on their way
  static_assert(!NORM || STAGED, "rows that await their norm are staged through LDS");
  constexpr bool FAST = STAGED;
  [[maybe_unused]] bf16x8_t fn[FAST ? KSTEPS : 1];
  [[maybe_unused]] const bool inside = (int)(blockIdx.y * NW + wave + 1) * (KSTEPS * 32) <= K;
  [[maybe_unused]] auto load_first = [&](auto first, auto last) {
    const int wrow = min((int)(blockIdx.x * groups_per_block) * 16 + frag_row, N - 1);
    const bf16_t* wp = W + (size_t)wrow * K + kbase;
#pragma unroll
    for (int s = first; s < last; ++s) fn[s] = *reinterpret_cast<const bf16x8_t*>(wp + s * 32);
  };
  constexpr std::integral_constant<int, 0> S0{};
  constexpr std::integral_constant<int, KSTEPS / 2> S1{};
  constexpr std::integral_constant<int, KSTEPS> S2{};
  [[maybe_unused]] bf16_t* staged = reinterpret_cast<bf16_t*>(rows16_staged);
  if constexpr (NORM && STAGED) {
    // the rows take a quarter of the registers while they are on their way: the whole
    // first group is requested with them
    stage_normed_rows<NW, KSTEPS, 16>(xa, normed.x, normed.rows, normed.weight, M, K, tid, ssw,
                                      staged, [&]() { load_first(S0, S2); });
  } else if constexpr (STAGED) {
    if (inside) {
      bf16_t* mine = staged + (size_t)wave * rows16_stage_places(M) * ROWS16_STAGE_STRIDE;
      const int kslice = (blockIdx.y * NW + wave) * KSTEPS * 32;
      if constexpr (MERGED) {
        if (merged.nsplit <= 2)
          stage_merged_rows<KSTEPS, 2>(xa, merged, M, K, kslice, mine, lane, [&]() { load_first(S0, S2); });
        else if (merged.nsplit <= 4)
          stage_merged_rows<KSTEPS, 4>(xa, merged, M, K, kslice, mine, lane, [&]() { load_first(S0, S2); });
        else if (merged.nsplit <= 8)
          stage_merged_rows<KSTEPS, 8>(xa, merged, M, K, kslice, mine, lane, [&]() { load_first(S0, S2); });
        else
          stage_merged_rows<KSTEPS, 16>(xa, merged, M, K, kslice, mine, lane, [&]() { load_first(S0, S2); });
      } else {
        stage_rows<KSTEPS>(xa, A, M, K, kslice, mine, lane, [&]() { load_first(S0, S2); });
      }
    } else {
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) xa[s] = zero8;
    }
  } else {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      xa[s] = (frag_row < M && k < K)
                  ? *reinterpret_cast<const bf16x8_t*>(A + (size_t)frag_row * K + k) : zero8;
    }
  }

  const bool partial = gridDim.y > 1 && !accumulate;
  // One row group; `more` (a compile-time flag): another group of this workgroup follows.
  auto row_group = [&](int g, auto more, auto burst) {
    const int n0 = (blockIdx.x * groups_per_block + g) * 16;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    if constexpr (FAST) {
      if (inside) {
        if constexpr (decltype(burst)::value) {
          if (g > 0) {
            const bf16_t* wp = W + (size_t)min(n0 + frag_row, N - 1) * K + kbase;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) fn[s] = *reinterpret_cast<const bf16x8_t*>(wp + s * 32);
            __builtin_amdgcn_sched_barrier(0);   // every load is requested before the first product
          }
        }
        // `more`: the next row group's fragments are requested one by one into the registers
        // that the products free, so the wave's requests to memory never run dry between groups
        [[maybe_unused]] const bf16_t* nxt =
            W + (size_t)min(n0 + 16 + frag_row, N - 1) * K + kbase;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fn[s], xa[s], acc, 0, 0, 0);
          if constexpr (decltype(more)::value) {
            fn[s] = *reinterpret_cast<const bf16x8_t*>(nxt + s * 32);
            __builtin_amdgcn_sched_barrier(0);   // in this order: the compiler would bunch the loads
          }
        }
      }
    } else {
      const int wrow = n0 + frag_row;
      const bool wvalid = wrow < N;
      const bf16_t* wp = W + (size_t)(wvalid ? wrow : 0) * K + kbase;
      // all of a row group's weight fragments (HALF of them when a wave's K slice is
      // long) are requested before the first is used
#pragma unroll
      for (int h = 0; h < KSTEPS; h += HALF) {
        bf16x8_t fw[HALF];
#pragma unroll
        for (int s = 0; s < HALF; ++s) {
          const int k = kbase + (h + s) * 32;
          fw[s] = (wvalid && k < K) ? *reinterpret_cast<const bf16x8_t*>(wp + (h + s) * 32) : zero8;
        }
#pragma unroll
        for (int s = 0; s < HALF; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[s], xa[h + s], acc, 0, 0, 0);
      }
    }
    if (NW > 1) {
      float* mine = red[g & 1][wave][lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[r] = acc[r];
      __syncthreads();
    }
    if (wave == 0) {
      const int m = lane & 15, nn = n0 + (lane >> 4) * 4;
      if (m < M) {
        float scale = 1.f;
        if constexpr (NORM) scale = normed_row_scale<NW>(ssw, m, K, normed.eps);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = nn + r;
          if (n >= N) continue;
          float v = acc[r];
          if (NW > 1) {
            v = red[g & 1][0][lane][r];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += red[g & 1][w][lane][r];
          }
          if constexpr (NORM) v *= scale;
          if (bias && blockIdx.y == 0) v += bias[n];
          if (accumulate)
            unsafeAtomicAdd(reinterpret_cast<float*>(C) + (size_t)m * N + n, v);
          else if (partial)
            reinterpret_cast<float*>(C)[((size_t)blockIdx.y * M + m) * N + n] = v;
          else
            C[(size_t)m * N + n] = from_f32<TC>(v);
        }
      }
    }
  };
  // the row groups of this workgroup that lie inside N (at least one: the grid is made so)
  const int first = blockIdx.x * groups_per_block;
  const int count = min(groups_per_block, (N + 15) / 16 - first);
  // ROLL (two groups a workgroup): the second is requested while the first is multiplied.
  // With more (the output head: two workgroups a compute unit take turns) a group requested
  // whole before its products measured faster (8 rows, 65536 x 2048: 52.5 against 53.8 us).
  if constexpr (ROLL) {
    int g = 0;
    for (; g + 1 < count; ++g) row_group(g, std::true_type{}, std::false_type{});
    row_group(g, std::false_type{}, std::false_type{});
  } else {
    for (int g = 0; g < count; ++g) row_group(g, std::false_type{}, std::true_type{});
  }
}

// The ShortConv mixer's in_proj for a decode batch in which every request brings one
// token, with the mixer's gated convolution in the epilogue
// (/root/reference/src/cuda/layer_kernels.cu:192-222 folds convolution, activation and
// state into one kernel too).  W = [B rows (H); C rows (H); x rows (H)], rows of K.  A
// workgroup takes CH channels (4, 8 or 16: the launcher chooses so that about 256
// workgroups run) and with them 3 * CH weight rows, B then C then x of its channels, in
// TILES = ceil(3 * CH / 16) tiles of 16 (a lane reads whatever row its fragment names,
// so nothing is laid out anew; rows beyond 3 * CH repeat addresses that other lanes ask
// for).  The tiles' sums, scaled and rounded as the projection would store them, meet in
// LDS, and wave 0 does what short_conv_kernel's head threads do, with the same operations
// in the same order, lane (m, q) for token m and the channels q * CH / 4 ... of the CH:
//   u = B * x;  the state's L values move up by one and take u;  c = bias + sum_j w[j] * state[j];
//   y = C * c
// Slot, state and filter are requested at the kernel's start, so they have arrived when
// the products are done.  Rows come as NormedRows, staged through LDS.
template <int NW, int TILES, int MAX_ROWS>
__global__ void __launch_bounds__(NW * 64, 2)
gemm_bf16_rows16_gated_conv_kernel(NormedRowsArg normed, const bf16_t* __restrict__ W,
                                   const float* __restrict__ taps,
                                   const float* __restrict__ conv_bias, float* __restrict__ state,
                                   long long slot_stride, const int* __restrict__ slot_id,
                                   bf16_t* __restrict__ y, int M, int H, int K, int L) {
  constexpr int KSTEPS = 16, MAXL = 8;
  constexpr int CH = TILES == 1 ? 4 : (TILES == 2 ? 8 : 16);
  constexpr int PER = CH / 4;                       // channels of a lane in the epilogue
  __shared__ float red[2][NW][64][4];
  __shared__ float ssw[NW][16];
  __shared__ float zs[TILES * 16][16 + 1];   // [weight row of the workgroup][token]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const int kbase = wave * KSTEPS * 32 + frag_k;
  const bool inside = (wave + 1) * (KSTEPS * 32) <= K;
  const int c0 = blockIdx.x * CH;
  // the weight row of this lane's fragment in tile t: row v = t * 16 + frag_row of the
  // workgroup's 3 * CH (a row beyond them takes the place of one CH earlier)
  auto weight_row = [&](int t) {
    int v = t * 16 + frag_row;
    if (v >= 3 * CH) v -= CH;
    return W + (size_t)((v / CH) * H + c0 + v % CH) * K + kbase;
  };

  // wave 0: token m, channels ch .. ch + PER - 1
  const int m = lane & 15, ch = c0 + (lane >> 4) * PER;
  const bool mine = wave == 0 && m < M;
  float hist[MAXL][PER], wt[MAXL][PER], cb[PER];
  float* st = nullptr;
  // (up to eight rows: before the rows are staged, so that the two trips to memory, slot
  // then state, are over when the products are; with more rows the staging needs the
  // registers, and the products take long enough for the loads to follow it)
  auto request_state = [&]() {
    if (mine) {
      st = state + (size_t)slot_id[m] * (size_t)slot_stride + (size_t)ch * L;
#pragma unroll
      for (int j = 0; j < MAXL; ++j)
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          hist[j][i] = j < L ? st[i * L + j] : 0.f;
          wt[j][i] = j < L ? taps[(size_t)j * H + ch + i] : 0.f;
        }
#pragma unroll
      for (int i = 0; i < PER; ++i) cb[i] = conv_bias ? conv_bias[ch + i] : 0.f;
    }
  };
  if constexpr (MAX_ROWS <= ROWS16_STAGE_ROWS) request_state();

  bf16x8_t xa[KSTEPS], fn[KSTEPS];
  stage_normed_rows<NW, KSTEPS, MAX_ROWS>(xa, normed.x, normed.rows, normed.weight, M, K, tid,
                                          ssw, reinterpret_cast<bf16_t*>(rows16_staged), [&]() {
                                            const bf16_t* wp = weight_row(0);
#pragma unroll
                                            for (int s = 0; s < KSTEPS; ++s)
                                              fn[s] = *reinterpret_cast<const bf16x8_t*>(wp + s * 32);
                                          });
  if constexpr (MAX_ROWS > ROWS16_STAGE_ROWS) request_state();
  // One tile; `more` (a compile-time flag): the next tile's fragments are requested into
  // the registers that the products free.
  auto tile = [&](int t, auto more) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    if (inside) {
      if constexpr (decltype(more)::value) {
        const bf16_t* nxt = weight_row(t + 1);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fn[s], xa[s], acc, 0, 0, 0);
          fn[s] = *reinterpret_cast<const bf16x8_t*>(nxt + s * 32);
          __builtin_amdgcn_sched_barrier(0);   // in this order: the compiler would bunch the loads
        }
      } else {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fn[s], xa[s], acc, 0, 0, 0);
      }
    }
    if (NW > 1) {
      float* mine_red = red[t & 1][wave][lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) mine_red[r] = acc[r];
      __syncthreads();
    }
    if (wave == 0 && m < M) {
      const float scale = normed_row_scale<NW>(ssw, m, K, normed.eps);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[r];
        if (NW > 1) {
          v = red[t & 1][0][lane][r];
#pragma unroll
          for (int w = 1; w < NW; ++w) v += red[t & 1][w][lane][r];
        }
        zs[t * 16 + (lane >> 4) * 4 + r][m] = (float)(bf16_t)(v * scale);
      }
    }
  };
  if constexpr (TILES >= 2) tile(0, std::true_type{});
  if constexpr (TILES >= 3) tile(1, std::true_type{});
  tile(TILES - 1, std::false_type{});
  if (!mine) return;
  // (wave 0 reads what its own lanes wrote: LDS operations of one wave run in order)
  bf16_t out[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = (lane >> 4) * PER + i;
    const float u = zs[c][m] * zs[2 * CH + c][m];
#pragma unroll
    for (int j = 0; j < MAXL - 1; ++j)
      if (j < L - 1) hist[j][i] = hist[j + 1][i];
#pragma unroll
    for (int j = 0; j < MAXL; ++j)
      if (j == L - 1) hist[j][i] = u;
    float acc = cb[i];
#pragma unroll
    for (int j = 0; j < MAXL; ++j)
      if (j < L) acc = fmaf(wt[j][i], hist[j][i], acc);
    out[i] = (bf16_t)(zs[CH + c][m] * acc);
#pragma unroll
    for (int j = 0; j < MAXL; ++j)
      if (j < L) st[i * L + j] = hist[j][i];
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) y[(size_t)m * H + ch + i] = out[i];
}

// The same kernel for the fused gate|up projection of a SwiGLU feed-forward,
// W = [gate rows (I); up rows (I)]: a workgroup computes a row group of the gate
// and the matching row group of the up projection and writes
//   C[m, n] = silu(gate[m, n]) * up[m, n],   silu(g) = g / (1 + exp(-g)),
// from the 32-bit accumulators (/root/reference/src/transformer/ffn.zig:24-30), so
// the [M, 2I] intermediate never goes to memory.  K is not split over workgroups.
template <int NW, int KSTEPS, bool NORM, bool STAGED>
__global__ void __launch_bounds__(NW * 64, 2)
gemm_bf16_rows16_swiglu_kernel(const bf16_t* __restrict__ A, NormedRowsArg normed,
                               const bf16_t* __restrict__ W, bf16_t* __restrict__ C, int M, int I,
                               int K, int groups_per_block) {
  __shared__ float red[2][2][NW][64][4];
  __shared__ float ssw[NW][16];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const int kbase = wave * KSTEPS * 32 + frag_k;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int CHUNK = KSTEPS > 8 ? 8 : KSTEPS;   // fragments of each operand in flight

  bf16x8_t xa[KSTEPS];
  // NORM: as in gemm_bf16_rows16_kernel, with all of a row group's gate and up rows in
  // registers; the first group's first quarter is requested with the rows (whose 32-bit
  // values fill half of the registers meanwhile), the rest once they are converted
  [[maybe_unused]] bf16x8_t ng[NORM ? KSTEPS : 1], nu[NORM ? KSTEPS : 1];
  [[maybe_unused]] const bool inside = (wave + 1) * (KSTEPS * 32) <= K;
  [[maybe_unused]] auto load_steps = [&](int g, auto first, auto last) {
    const int wrow = min((int)(blockIdx.x * groups_per_block + g) * 16 + frag_row, I - 1);
    const bf16_t* gp = W + (size_t)wrow * K + kbase;
    const bf16_t* up = gp + (size_t)I * K;
#pragma unroll
    for (int s = first; s < last; ++s) {
      ng[s] = *reinterpret_cast<const bf16x8_t*>(gp + s * 32);
      nu[s] = *reinterpret_cast<const bf16x8_t*>(up + s * 32);
    }
  };
  constexpr std::integral_constant<int, 0> S0{};
  constexpr std::integral_constant<int, KSTEPS / 2> S1{};
  constexpr std::integral_constant<int, KSTEPS> S2{};
  [[maybe_unused]] bf16_t* staged = reinterpret_cast<bf16_t*>(rows16_staged);
  if constexpr (NORM && STAGED) {
    // (the rows take a quarter of the registers on their way: half of the first group
    // is requested with them)
    stage_normed_rows<NW, KSTEPS, 16>(xa, normed.x, normed.rows, normed.weight, M, K, tid, ssw,
                                      staged, [&]() { load_steps(0, S0, S1); });
  } else if constexpr (STAGED) {
    stage_rows<KSTEPS>(xa, A, M, K, wave * KSTEPS * 32,
                       staged + (size_t)wave * rows16_stage_places(M) * ROWS16_STAGE_STRIDE, lane, []() {});
  } else {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int k = kbase + s * 32;
      xa[s] = (frag_row < M && k < K)
                  ? *reinterpret_cast<const bf16x8_t*>(A + (size_t)frag_row * K + k) : zero8;
    }
  }

  if constexpr (NORM) {
    if (inside) {
      load_steps(0, S1, S2);
      __builtin_amdgcn_sched_barrier(0);   // every load is requested before the first product
    }
  }
  // One row group; `more` (a compile-time flag): another group of this workgroup follows.
  auto row_group = [&](int g, auto more, auto burst) {
    const int n0 = (blockIdx.x * groups_per_block + g) * 16;
    f32x4_t ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
    if constexpr (NORM) {
      if (inside) {
        if constexpr (decltype(burst)::value) {
          if (g > 0) {
            load_steps(g, S0, S2);
            __builtin_amdgcn_sched_barrier(0);   // every load is requested before the first product
          }
        }
        // `more`: the next row group's fragments are requested one by one into the registers
        // that the products free, so the wave's requests to memory never run dry between groups
        [[maybe_unused]] const bf16_t* ngp =
            W + (size_t)min(n0 + 16 + frag_row, I - 1) * K + kbase;
        [[maybe_unused]] const bf16_t* nup = ngp + (size_t)I * K;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          ag = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ng[s], xa[s], ag, 0, 0, 0);
          au = __builtin_amdgcn_mfma_f32_16x16x32_bf16(nu[s], xa[s], au, 0, 0, 0);
          if constexpr (decltype(more)::value) {
            ng[s] = *reinterpret_cast<const bf16x8_t*>(ngp + s * 32);
            nu[s] = *reinterpret_cast<const bf16x8_t*>(nup + s * 32);
            __builtin_amdgcn_sched_barrier(0);   // in this order: the compiler would bunch the loads
          }
        }
      }
    } else {
      const int wrow = n0 + frag_row;
      const bool wvalid = wrow < I;
      const bf16_t* gp = W + (size_t)(wvalid ? wrow : 0) * K + kbase;
      const bf16_t* up = gp + (size_t)I * K;
#pragma unroll
      for (int h = 0; h < KSTEPS; h += CHUNK) {
        bf16x8_t fg[CHUNK], fu[CHUNK];
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
          const bool ok = wvalid && kbase + (h + s) * 32 < K;
          fg[s] = ok ? *reinterpret_cast<const bf16x8_t*>(gp + (h + s) * 32) : zero8;
          fu[s] = ok ? *reinterpret_cast<const bf16x8_t*>(up + (h + s) * 32) : zero8;
        }
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
          ag = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fg[s], xa[h + s], ag, 0, 0, 0);
          au = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fu[s], xa[h + s], au, 0, 0, 0);
        }
      }
    }
    if (NW > 1) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        red[g & 1][0][wave][lane][r] = ag[r];
        red[g & 1][1][wave][lane][r] = au[r];
      }
      __syncthreads();
    }
    if (wave == 0) {
      const int m = lane & 15, nn = n0 + (lane >> 4) * 4;
      if (m < M) {
        float scale = 1.f;
        if constexpr (NORM) scale = normed_row_scale<NW>(ssw, m, K, normed.eps);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = nn + r;
          if (n >= I) continue;
          float gv = ag[r], uv = au[r];
          if (NW > 1) {
            gv = red[g & 1][0][0][lane][r];
            uv = red[g & 1][1][0][lane][r];
#pragma unroll
            for (int w = 1; w < NW; ++w) {
              gv += red[g & 1][0][w][lane][r];
              uv += red[g & 1][1][w][lane][r];
            }
          }
          if constexpr (NORM) {
            gv *= scale;
            uv *= scale;
          }
          C[(size_t)m * I + n] = (bf16_t)(gv * (1.0f / (1.0f + expf(-gv))) * uv);
        }
      }
    }
  };
  // the row groups of this workgroup that lie inside I (at least one: the grid is made so)
  const int first = blockIdx.x * groups_per_block;
  const int count = min(groups_per_block, (I + 15) / 16 - first);
  int g = 0;
  for (; g + 1 < count; ++g) row_group(g, std::true_type{}, std::false_type{});
  row_group(g, std::false_type{}, std::false_type{});
}

// `normed` (with normed->x set) replaces the bfloat16 activations `a` by rows of the
// 32-bit stream that the kernel normalises itself; it needs one workgroup to cover K
// with 16 steps a wave (K <= 4096, a multiple of 512) and K not split over workgroups.
// A workgroup may ask for 64 KB of LDS at launch; a kernel that wants more (eight waves
// staging eight rows) is told so once.  The kernels are few: a short list remembers them.
static int rows16_allow_lds(const void* kernel, size_t bytes) {
  if (bytes <= 48 * 1024) return 0;
  static std::mutex guard;
  static std::vector<const void*> allowed;
  std::lock_guard<std::mutex> lock(guard);
  for (const void* k : allowed)
    if (k == kernel) return 0;
  const hipError_t rc =
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
  if (rc != hipSuccess) {
    (void)hipGetLastError();
    return (int)rc;
  }
  allowed.push_back(kernel);
  return 0;
}

// Only in a build made for tuning runs (-DZA_TUNING_BUILD): row groups per workgroup of
// the decode products that take no such argument (0: the launchers choose).  The
// library the engine loads has no such switch: nothing process-wide steers its launches.
#ifdef ZA_TUNING_BUILD
static int rows16_groups_override = 0;
extern "C" void za_gemm_rows16_set_groups_per_block(int groups) { rows16_groups_override = groups; }
#else
static constexpr int rows16_groups_override = 0;
#endif

static bool rows16_takes_norm(int K, int ksplit) {
  return ksplit == 1 && K <= 4096 && K % 512 == 0;
}

static int launch_rows16(const bf16_t* a, const NormedRowsArg* normed, const bf16_t* w,
                         const float* bias, void* C, int c_dtype, int M, int N, int K, int ksplit,
                         int accumulate, hipStream_t stream, int groups_per_block = 0,
                         const MergedRowsArg* merged_rows = nullptr) {
  if (ksplit < 1 || (ksplit > 1 && (c_dtype != 0 || K % (ksplit * 32) != 0))) return ZA_ERR_ARG;
  if (accumulate && c_dtype != 0) return ZA_ERR_ARG;
  const bool norm = normed && normed->x;
  if (norm && (!normed->weight || !rows16_takes_norm(K, ksplit))) return ZA_ERR_UNSUPPORTED;
  const bool merge = merged_rows && merged_rows->acc;
  if (merge && (norm || c_dtype != 0 || M > ROWS16_STAGE_ROWS || K % 512 != 0 || merged_rows->nsplit > 16 ||
                merged_rows->nsplit < 1 || merged_rows->d % 8 != 0 || K % merged_rows->d != 0 ||
                K / ksplit % 512 != 0 || K / ksplit > 4096))
    return ZA_ERR_UNSUPPORTED;
  if (!norm && !a && !merge) return ZA_ERR_ARG;
  const int kper = (K + ksplit - 1) / ksplit;   // K range of one workgroup
  if (kper > 8192) return ZA_ERR_UNSUPPORTED;
  const int groups = (N + 15) / 16;
  // Measured at M = 8 on one MI355X: every shape runs at about 4.8 TB/s plus about
  // 3 us; with many row groups, several per workgroup re-read the activations less
  // often, with few, one per workgroup keeps every compute unit loading.
  int per_block = 1;
  if (groups >= 2048) per_block = 8;
  else if (groups >= 768) per_block = 2;
  // with the norm in the kernel every workgroup prepares the step's rows first: two row
  // groups share that from 384 groups on (8 rows: in_proj 10.7 -> 9.1 us)
  if (norm && per_block == 1 && groups >= 384) per_block = 2;
  if (rows16_groups_override > 0) per_block = rows16_groups_override;
  if (groups_per_block > 0) per_block = groups_per_block;
  dim3 grid((groups + per_block - 1) / per_block, ksplit);
  const NormedRowsArg none = {nullptr, nullptr, nullptr, 0.f};
  const MergedRowsArg unmerged = {nullptr, nullptr, 0, 0};
  // the rows go through LDS (16 steps a wave only; without the norm: only where K is a
  // multiple of a wave's slice, the condition of the kernel's loads without conditions)
  const bool stage = norm || K % 512 == 0;
#define ZA_R16_LAUNCH(NW, KS, TC, NORM, STAGED, ROLL)                                         \
  {                                                                                           \
    const size_t lds = STAGED ? rows16_stage_bytes(NW, M) : 0;                                \
    auto kernel = gemm_bf16_rows16_kernel<NW, KS, TC, NORM, STAGED, ROLL>;                    \
    if (const int rc = rows16_allow_lds((const void*)kernel, lds)) return rc;                         \
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds, stream, a, NORM ? *normed : none, w, \
                       bias, (TC*)C, M, N, K, per_block, accumulate, unmerged);               \
  }
#define ZA_R16_MERGED(NW, KS, ROLL)                                                           \
  {                                                                                           \
    const size_t lds = rows16_stage_bytes(NW, M);                                             \
    auto kernel = gemm_bf16_rows16_kernel<NW, KS, float, false, true, ROLL, true>;            \
    if (const int rc = rows16_allow_lds((const void*)kernel, lds)) return rc;                 \
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds, stream, a, none, w, bias, (float*)C, \
                       M, N, K, per_block, accumulate, *merged_rows);                         \
  }
#define ZA_R16_TYPES(NW, KS, NORM, STAGED, ROLL)                                              \
  {                                                                                           \
    if (c_dtype == 0) ZA_R16_LAUNCH(NW, KS, float, NORM, STAGED, ROLL)                        \
    else ZA_R16_LAUNCH(NW, KS, bf16_t, NORM, STAGED, ROLL)                                    \
  }
#define ZA_R16_ROLL(NW, KS, NORM)                                                             \
  {                                                                                           \
    if (per_block <= 2) ZA_R16_TYPES(NW, KS, NORM, true, true)                                \
    else ZA_R16_TYPES(NW, KS, NORM, true, false)                                              \
  }
#define ZA_R16_CASE(NW, KS)                                                                   \
  {                                                                                           \
    if constexpr (KS == 16) {                                                                 \
      if (merge) {                                                                            \
        if (per_block <= 2) ZA_R16_MERGED(NW, KS, true)                                       \
        else ZA_R16_MERGED(NW, KS, false)                                                     \
      } else                                                                                  \
      if (norm) ZA_R16_ROLL(NW, KS, true)                                                     \
      else if (stage) ZA_R16_ROLL(NW, KS, false)                                              \
      else ZA_R16_TYPES(NW, KS, false, false, false)                                          \
    } else {                                                                                  \
      if (norm) return ZA_ERR_UNSUPPORTED;                                                    \
      ZA_R16_TYPES(NW, KS, false, false, false)                                               \
    }                                                                                         \
    return za_launch_status();                                                                \
  }
  if (kper <= 512) ZA_R16_CASE(1, 16)
  if (kper <= 1024) ZA_R16_CASE(2, 16)
  if (kper <= 2048) ZA_R16_CASE(4, 16)
  if (kper <= 4096) ZA_R16_CASE(8, 16)
  ZA_R16_CASE(8, 32)
#undef ZA_R16_CASE
#undef ZA_R16_ROLL
#undef ZA_R16_TYPES
#undef ZA_R16_LAUNCH
#undef ZA_R16_MERGED
}

// ------------------------------------------------------------------ launchers
// dtype codes: 0 = float32, 1 = bfloat16
extern "C" int za_gemm_f32(const void* A, int a_dtype, const float* W, const float* bias, void* C,
                           int c_dtype, int M, int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K <= 0 || !A || !W || !C) return ZA_ERR_ARG;
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM), block(256);
#define ZA_F32_CASE(AD, TA, CD, TC)                                                     \
  if (a_dtype == AD && c_dtype == CD) {                                                 \
    hipLaunchKernelGGL((gemm_f32_kernel<TA, TC>), grid, block, 0, stream, (const TA*)A, W, \
                       bias, (TC*)C, M, N, K);                                          \
    return za_launch_status();                                                          \
  }
  ZA_F32_CASE(0, float, 0, float)
  ZA_F32_CASE(1, bf16_t, 0, float)
  ZA_F32_CASE(1, bf16_t, 1, bf16_t)
  ZA_F32_CASE(0, float, 1, bf16_t)
#undef ZA_F32_CASE
  return ZA_ERR_UNSUPPORTED;
}

extern "C" int za_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int c_dtype,
                            int M, int N, int K, int force_tiled, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K <= 0 || !A || !W || !C) return ZA_ERR_ARG;
  if (K % 8 != 0) return ZA_ERR_UNSUPPORTED;  // rows must start on 16-byte boundaries
  if (c_dtype != 0 && c_dtype != 1) return ZA_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  if (M <= 16 && K <= 8192 && !force_tiled)
    return launch_rows16(a, nullptr, w, bias, C, c_dtype, M, N, K, 1, 0, stream);
  if (M <= 64 && !force_tiled) {
    dim3 grid((N + 15) / 16), block(256);
    const int mt = (M + 15) / 16;
#define ZA_SK_CASE(MT)                                                                        \
  if (mt == MT) {                                                                             \
    if (c_dtype == 0)                                                                         \
      hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, float>), grid, block, 0, stream, a, w,  \
                         bias, (float*)C, M, N, K);                                           \
    else                                                                                      \
      hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, bf16_t>), grid, block, 0, stream, a, w, \
                         bias, (bf16_t*)C, M, N, K);                                          \
    return za_launch_status();                                                                \
  }
    ZA_SK_CASE(1)
    ZA_SK_CASE(2)
    ZA_SK_CASE(3)
    ZA_SK_CASE(4)
#undef ZA_SK_CASE
  }
  dim3 grid((N + MF_BN - 1) / MF_BN, (M + MF_BM - 1) / MF_BM), block(256);
  if (c_dtype == 0)
    hipLaunchKernelGGL((gemm_bf16_mfma_kernel<float>), grid, block, 0, stream, a, w, bias,
                       (float*)C, M, N, K);
  else
    hipLaunchKernelGGL((gemm_bf16_mfma_kernel<bf16_t>), grid, block, 0, stream, a, w, bias,
                       (bf16_t*)C, M, N, K);
  return za_launch_status();
}

// The decode kernel with K split over workgroups: 32-bit partial results
// [ksplit][M][N] go into C (c_dtype must then be float32 and K a multiple of 32 * ksplit).
// `groups_per_block` overrides the launcher's choice of row groups per workgroup
// (0 leaves it to the launcher).
extern "C" int za_gemm_bf16_rows16(const void* A, const void* W, const float* bias, void* C,
                                   int c_dtype, int M, int N, int K, int ksplit,
                                   int groups_per_block, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K <= 0 || !A || !W || !C) return ZA_ERR_ARG;
  if (M > 16 || K % 8 != 0 || (c_dtype != 0 && c_dtype != 1)) return ZA_ERR_UNSUPPORTED;
  return launch_rows16((const bf16_t*)A, nullptr, (const bf16_t*)W, bias, C, c_dtype, M, N, K,
                       ksplit, 0, stream, groups_per_block);
}

// The decode kernel between two states of the 32-bit residual stream.
//   input:  bfloat16 activations A [M, K], or (A null) rows of the stream `x`
//           ([*, K] 32-bit; row m of the product is row rows[m], or m without `rows`)
//           that the kernel passes through an RMSNorm (norm_weight [K], eps) itself;
//           that needs K <= 4096, K % 512 == 0 and ksplit == 1;
//   output: stored to C [M, N] (c_dtype), or with `accumulate` added to the 32-bit
//           C [M, N] with atomics, K cut into `ksplit` ranges that all add there.
// Without `accumulate`, ksplit must be 1.
extern "C" int za_gemm_bf16_rows16_stream(const void* A, const float* x, const int* rows,
                                          const float* norm_weight, float eps, const void* W,
                                          const float* bias, void* C, int c_dtype, int M, int N,
                                          int K, int ksplit, int accumulate, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K <= 0 || !W || !C || (!A && !x)) return ZA_ERR_ARG;
  if (M > 16 || K % 8 != 0 || (c_dtype != 0 && c_dtype != 1)) return ZA_ERR_UNSUPPORTED;
  if (!accumulate && ksplit != 1) return ZA_ERR_ARG;
  const NormedRowsArg normed = {A ? nullptr : x, rows, norm_weight, eps};
  return launch_rows16((const bf16_t*)A, &normed, (const bf16_t*)W, bias, C, c_dtype, M, N, K,
                       ksplit, accumulate ? 1 : 0, stream);
}

// The decode kernel on rows that are an attention's output still in the partial results of
// `nsplit` context ranges (part_acc [M][K / d][nsplit][d], part_ml [M][K / d][nsplit][2], as
// za_paged_attention_decode_mfma leaves them): merged on the way in as
// attention_combine_kernel would, then multiplied and added to (or stored in) the 32-bit C.
// M <= 8, nsplit <= 16, K and K / ksplit multiples of 512.
extern "C" int za_gemm_bf16_rows16_merged(const float* part_acc, const float* part_ml, int nsplit,
                                          int d, const void* W, void* C, int M, int N, int K,
                                          int ksplit, int accumulate, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  if (M < 0 || N < 0 || K <= 0 || !W || !C || !part_acc || !part_ml || d <= 0) return ZA_ERR_ARG;
  if (!accumulate && ksplit != 1) return ZA_ERR_ARG;
  const MergedRowsArg merged = {part_acc, part_ml, nsplit, d};
  return launch_rows16(nullptr, nullptr, (const bf16_t*)W, nullptr, C, 0, M, N, K, ksplit,
                       accumulate ? 1 : 0, stream, 0, &merged);
}

// Fused gate|up projection with the SwiGLU gate applied to the accumulators:
// W is [2 * I, K] (gate rows, then up rows), C is bfloat16 [M, I], M <= 16, K <= 8192.
// The input is bfloat16 A [M, K], or (A null) rows of the 32-bit stream `x` that the
// kernel passes through an RMSNorm itself (K <= 4096, K % 512 == 0), as
// za_gemm_bf16_rows16_stream.
extern "C" int za_gemm_bf16_rows16_swiglu(const void* A, const float* x, const int* rows,
                                          const float* norm_weight, float eps, const void* W,
                                          void* C, int M, int I, int K, hipStream_t stream) {
  if (M == 0 || I == 0) return 0;
  if (M < 0 || I < 0 || K <= 0 || !W || !C || (!A && !x)) return ZA_ERR_ARG;
  if (M > 16 || K % 8 != 0 || K > 8192) return ZA_ERR_UNSUPPORTED;
  const bool norm = !A;
  if (norm && (!norm_weight || !rows16_takes_norm(K, 1))) return ZA_ERR_UNSUPPORTED;
  const NormedRowsArg normed = {norm ? x : nullptr, rows, norm_weight, eps};
  const int groups = (I + 15) / 16;
  // (with the norm in the kernel two row groups share the preparation of the step's rows:
  // 8 rows, I = 8192: 18.1 -> 16.9 us)
  int per_block = groups >= 2048 ? 4 : (norm && groups >= 384 ? 2 : 1);
  if (rows16_groups_override > 0) per_block = rows16_groups_override;
  dim3 grid((groups + per_block - 1) / per_block);
#define ZA_SG_LAUNCH(NW, KS, NORM, STAGED)                                                    \
  {                                                                                           \
    const size_t lds = STAGED ? rows16_stage_bytes(NW, M) : 0;                                \
    auto kernel = gemm_bf16_rows16_swiglu_kernel<NW, KS, NORM, STAGED>;                       \
    if (const int rc = rows16_allow_lds((const void*)kernel, lds)) return rc;                         \
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds, stream, (const bf16_t*)A, normed,    \
                       (const bf16_t*)W, (bf16_t*)C, M, I, K, per_block);                     \
  }
#define ZA_SG_CASE(NW, KS)                                                                    \
  {                                                                                           \
    if constexpr (KS == 16) {                                                                 \
      if (norm) ZA_SG_LAUNCH(NW, KS, true, true) else ZA_SG_LAUNCH(NW, KS, false, true)       \
    } else {                                                                                  \
      if (norm) return ZA_ERR_UNSUPPORTED;                                                    \
      ZA_SG_LAUNCH(NW, KS, false, false)                                                      \
    }                                                                                         \
    return za_launch_status();                                                                \
  }
  if (K <= 512) ZA_SG_CASE(1, 16)
  if (K <= 1024) ZA_SG_CASE(2, 16)
  if (K <= 2048) ZA_SG_CASE(4, 16)
  if (K <= 4096) ZA_SG_CASE(8, 16)
  ZA_SG_CASE(8, 32)
#undef ZA_SG_CASE
#undef ZA_SG_LAUNCH
}

// The ShortConv mixer from the 32-bit stream to the convolution's output in one kernel
// (gemm_bf16_rows16_gated_conv_kernel), for a decode batch of M <= 16 requests with one
// token each: row m of the product is token m and belongs to the request whose state
// slot is slot_id[m].  W [3H, K] bfloat16 (B, C, x rows), taps [L, H] and conv_bias [H]
// (or null) 32-bit, state as za_short_conv takes it, y [M, H] bfloat16.  K a multiple of
// 512 up to 4096, H a multiple of 16, L <= 8.  `channels` (0: the launcher chooses) is
// the number of channels a workgroup takes: 4, 8 or 16.
extern "C" int za_gemm_bf16_rows16_gated_conv(const float* x, const int* rows,
                                              const float* norm_weight, float eps, const void* W,
                                              const float* taps, const float* conv_bias,
                                              float* state, long long slot_stride,
                                              const int* slot_id, void* y, int M, int H, int K,
                                              int L, int channels, hipStream_t stream) {
  if (M == 0 || H == 0) return 0;
  if (M < 0 || H < 0 || K <= 0 || L <= 0 || !x || !norm_weight || !W || !taps || !state || !slot_id ||
      !y || slot_stride < (long long)H * L)
    return ZA_ERR_ARG;
  if (M > 16 || H % 16 != 0 || L > 8 || !rows16_takes_norm(K, 1))
    return ZA_ERR_UNSUPPORTED;
  if (channels != 0 && channels != 4 && channels != 8 && channels != 16) return ZA_ERR_ARG;
  // measured at 8 rows and at 1 (us; widths 1024, 1536, 2048, 2560, 4096):
  //   4 channels   5.1 / 4.4    7.8 / 6.7    9.8 / 8.1   17.5 / 14.8   34.8 / 26.2
  //   8            6.5 / 5.8    8.0 / 7.3    9.5 / 9.0   18.2 / 16.2   28.5 / 24.6
  //   16           7.7 / 6.9    9.6 / 8.8   11.0 / 10.9  14.5 / 13.4   22.7 / 20.7
  if (channels == 0) channels = H <= 1536 ? 4 : (H <= 2048 ? (M <= 2 ? 4 : 8) : 16);
  const NormedRowsArg normed = {x, rows, norm_weight, eps};
  dim3 grid(H / channels);
#define ZA_GC_LAUNCH(NW, TILES)                                                               \
  {                                                                                           \
    const size_t lds = rows16_stage_bytes(NW, M);                                             \
    auto kernel = M <= ROWS16_STAGE_ROWS ? gemm_bf16_rows16_gated_conv_kernel<NW, TILES, 8>   \
                                         : gemm_bf16_rows16_gated_conv_kernel<NW, TILES, 16>; \
    if (const int rc = rows16_allow_lds((const void*)kernel, lds)) return rc;                 \
    hipLaunchKernelGGL(kernel, grid, dim3(NW * 64), lds, stream, normed, (const bf16_t*)W,    \
                       taps, conv_bias, state, slot_stride, slot_id, (bf16_t*)y, M, H, K, L); \
    return za_launch_status();                                                                \
  }
#define ZA_GC_CASE(NW)                                                                        \
  {                                                                                           \
    if (channels == 4) ZA_GC_LAUNCH(NW, 1)                                                    \
    if (channels == 8) ZA_GC_LAUNCH(NW, 2)                                                    \
    ZA_GC_LAUNCH(NW, 3)                                                                       \
  }
  if (K <= 512) ZA_GC_CASE(1)
  if (K <= 1024) ZA_GC_CASE(2)
  if (K <= 2048) ZA_GC_CASE(4)
  ZA_GC_CASE(8)
#undef ZA_GC_CASE
#undef ZA_GC_LAUNCH
}
