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
template <int NW, int KSTEPS, typename TC>
__global__ void __launch_bounds__(NW * 64)
gemm_bf16_rows16_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                        const float* __restrict__ bias, TC* __restrict__ C, int M, int N, int K,
                        int groups_per_block) {
  __shared__ float red[2][NW][64][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const int kbase = (blockIdx.y * NW + wave) * KSTEPS * 32 + frag_k;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int HALF = KSTEPS > 16 ? 16 : KSTEPS;   // weight fragments in flight at once

  bf16x8_t xa[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int k = kbase + s * 32;
    xa[s] = (frag_row < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(A + (size_t)frag_row * K + k)
                                    : zero8;
  }

  const bool partial = gridDim.y > 1;
  for (int g = 0; g < groups_per_block; ++g) {
    const int n0 = (blockIdx.x * groups_per_block + g) * 16;
    if (n0 >= N) break;
    const int wrow = n0 + frag_row;
    const bool wvalid = wrow < N;
    const bf16_t* wp = W + (size_t)(wvalid ? wrow : 0) * K + kbase;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
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
    if (NW > 1) {
      float* mine = red[g & 1][wave][lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[r] = acc[r];
      __syncthreads();
    }
    if (wave == 0) {
      const int m = lane & 15, nn = n0 + (lane >> 4) * 4;
      if (m < M) {
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
          if (bias && blockIdx.y == 0) v += bias[n];
          if (partial)
            reinterpret_cast<float*>(C)[((size_t)blockIdx.y * M + m) * N + n] = v;
          else
            C[(size_t)m * N + n] = from_f32<TC>(v);
        }
      }
    }
  }
}

// The same kernel for the fused gate|up projection of a SwiGLU feed-forward,
// W = [gate rows (I); up rows (I)]: a workgroup computes a row group of the gate
// and the matching row group of the up projection and writes
//   C[m, n] = silu(gate[m, n]) * up[m, n],   silu(g) = g / (1 + exp(-g)),
// from the 32-bit accumulators (/root/reference/src/transformer/ffn.zig:24-30), so
// the [M, 2I] intermediate never goes to memory.  K is not split over workgroups.
template <int NW, int KSTEPS>
__global__ void __launch_bounds__(NW * 64)
gemm_bf16_rows16_swiglu_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                               bf16_t* __restrict__ C, int M, int I, int K,
                               int groups_per_block) {
  __shared__ float red[2][2][NW][64][4];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
  const int kbase = wave * KSTEPS * 32 + frag_k;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int CHUNK = KSTEPS > 8 ? 8 : KSTEPS;   // fragments of each operand in flight

  bf16x8_t xa[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int k = kbase + s * 32;
    xa[s] = (frag_row < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(A + (size_t)frag_row * K + k)
                                    : zero8;
  }

  for (int g = 0; g < groups_per_block; ++g) {
    const int n0 = (blockIdx.x * groups_per_block + g) * 16;
    if (n0 >= I) break;
    const int wrow = n0 + frag_row;
    const bool wvalid = wrow < I;
    const bf16_t* gp = W + (size_t)(wvalid ? wrow : 0) * K + kbase;
    const bf16_t* up = gp + (size_t)I * K;
    f32x4_t ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
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
          C[(size_t)m * I + n] = (bf16_t)(gv * (1.0f / (1.0f + expf(-gv))) * uv);
        }
      }
    }
  }
}

static int launch_rows16(const bf16_t* a, const bf16_t* w, const float* bias, void* C, int c_dtype,
                         int M, int N, int K, int ksplit, hipStream_t stream,
                         int groups_per_block = 0) {
  if (ksplit < 1 || (ksplit > 1 && (c_dtype != 0 || K % (ksplit * 32) != 0))) return ZA_ERR_ARG;
  const int kper = (K + ksplit - 1) / ksplit;   // K range of one workgroup
  if (kper > 8192) return ZA_ERR_UNSUPPORTED;
  const int groups = (N + 15) / 16;
  // Measured at M = 8 on one MI355X: every shape runs at about 4.8 TB/s plus about
  // 3 us; with many row groups, several per workgroup re-read the activations less
  // often, with few, one per workgroup keeps every compute unit loading.
  int per_block = 1;
  if (groups >= 2048) per_block = 8;
  else if (groups >= 768) per_block = 2;
  if (groups_per_block > 0) per_block = groups_per_block;
  dim3 grid((groups + per_block - 1) / per_block, ksplit);
#define ZA_R16_CASE(NW, KS)                                                                   \
  {                                                                                           \
    dim3 block(NW * 64);                                                                      \
    if (c_dtype == 0)                                                                         \
      hipLaunchKernelGGL((gemm_bf16_rows16_kernel<NW, KS, float>), grid, block, 0,            \
                         stream, a, w, bias, (float*)C, M, N, K, per_block);                  \
    else                                                                                      \
      hipLaunchKernelGGL((gemm_bf16_rows16_kernel<NW, KS, bf16_t>), grid, block, 0,           \
                         stream, a, w, bias, (bf16_t*)C, M, N, K, per_block);                 \
    return za_launch_status();                                                                \
  }
  if (kper <= 512) ZA_R16_CASE(1, 16)
  if (kper <= 1024) ZA_R16_CASE(2, 16)
  if (kper <= 2048) ZA_R16_CASE(4, 16)
  if (kper <= 4096) ZA_R16_CASE(8, 16)
  ZA_R16_CASE(8, 32)
#undef ZA_R16_CASE
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
    return launch_rows16(a, w, bias, C, c_dtype, M, N, K, 1, stream);
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
  return launch_rows16((const bf16_t*)A, (const bf16_t*)W, bias, C, c_dtype, M, N, K, ksplit,
                       stream, groups_per_block);
}

// Fused gate|up projection with the SwiGLU gate applied to the accumulators:
// W is [2 * I, K] (gate rows, then up rows), C is bfloat16 [M, I], M <= 16, K <= 8192.
extern "C" int za_gemm_bf16_rows16_swiglu(const void* A, const void* W, void* C, int M, int I,
                                          int K, hipStream_t stream) {
  if (M == 0 || I == 0) return 0;
  if (M < 0 || I < 0 || K <= 0 || !A || !W || !C) return ZA_ERR_ARG;
  if (M > 16 || K % 8 != 0 || K > 8192) return ZA_ERR_UNSUPPORTED;
  const int groups = (I + 15) / 16;
  const int per_block = groups >= 2048 ? 4 : 1;
  dim3 grid((groups + per_block - 1) / per_block);
#define ZA_SG_CASE(NW, KS)                                                                    \
  {                                                                                           \
    hipLaunchKernelGGL((gemm_bf16_rows16_swiglu_kernel<NW, KS>), grid, dim3(NW * 64), 0,      \
                       stream, (const bf16_t*)A, (const bf16_t*)W, (bf16_t*)C, M, I, K,       \
                       per_block);                                                            \
    return za_launch_status();                                                                \
  }
  if (K <= 512) ZA_SG_CASE(1, 16)
  if (K <= 1024) ZA_SG_CASE(2, 16)
  if (K <= 2048) ZA_SG_CASE(4, 16)
  if (K <= 4096) ZA_SG_CASE(8, 16)
  ZA_SG_CASE(8, 32)
#undef ZA_SG_CASE
}
