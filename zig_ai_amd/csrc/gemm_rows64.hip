// bfloat16 matrix products of a step of 17 to 64 rows (a decode batch beyond the 16
// rows of gemm_bf16_rows16, a short portion of a prompt), with what surrounds them in a
// block fused in: the RMSNorm before the product, the SwiGLU gate behind it, the
// addition to the residual stream.  The reference sends every product to its vendor's
// library (/root/reference/src/matmul/root.zig:292-313) and runs norm, gate and addition
// as kernels of their own (/root/reference/src/cuda/layer_kernels.cu); at these row
// counts a step is a chain of short dependent kernels, and every kernel saved is a
// launch and two trips to memory less.
//
//   y [M, N] = x [M, K] . W [N, K]^T,   17 <= M <= 64 (any M from 1 runs)
//
// One workgroup of sixteen waves takes 64 weight rows (one tile) and one range of K,
// which it walks in spans of 512 elements.  Waves 0-7 multiply: wave 4 h + g owns the
// tile's g-th group of 16 weight rows and the h-th half of every span, reads its weights
// from memory straight into matrix-core operand registers (16 bytes a lane and step of 32
// elements of K, the fragments of two spans requested ahead) and keeps the sums of all of
// the step's rows, MB = ceil(M / 16) accumulators; the two halves' sums meet in LDS at the
// end.  Waves 8-15 only bring the step's rows: they read a span's rows from memory (whole
// lines, a wave 2 MB rows), turn them into bfloat16 operands (with the norm: multiply by
// the norm's weight, which lies in LDS, and add up the squares) and put them into one of
// two places in LDS, a span ahead of the multiplying waves; one barrier a span.  The
// rows' loads wait behind no weight (a wave's loads return in the order of their
// requests: staged by the multiplying waves themselves, a span of rows would queue behind
// every weight requested before it) and the weights' behind no row.  Up to 32 rows the
// staging waves hold two spans in flight in registers, beyond that one.  The workgroups
// of a die start their walk over K at different spans (see `rot` below).
//
// Forms (MODE):
//   STORE    y as bfloat16
//   SWIGLU   W = [gate rows (N); up rows (N)]: silu(x . Wg^T) * (x . Wu^T) as bfloat16
//            [M, N]; a multiplying wave's sixteen rows are eight gate rows and the eight
//            up rows of the same outputs, and the two halves meet by one lane exchange
//   ADD      y is added to the 32-bit tensor C (the residual stream) with atomics; K may
//            be cut into gridDim.y ranges, which all add there
// NORM: the rows are rows of the 32-bit stream awaiting an RMSNorm (weight, eps;
// /root/reference/src/transformer/norm.zig:6-33); the row's scale goes onto the sums:
//   y[m, n] = (1 / sqrt(mean_k(x[m, k]^2) + eps)) * sum_k W[n, k] * bf16(x[m, k] * weight[k])
// with the squares summed in 32-bit from the unrounded x (K is then one range).
#include <hip/hip_runtime.h>

#include <mutex>
#include <type_traits>
#include <vector>

#include "common.h"

namespace {

struct NormedRows64 {
  const float* x;        // [*, K] 32-bit rows
  const int* rows;       // row m of the product is row rows[m] of x (null: row m)
  const float* weight;   // [K]
  float eps;
};

constexpr int R64_CHUNK = 256;              // elements of K one multiplying wave takes at a time
constexpr int R64_STEPS = R64_CHUNK / 32;   // matrix-core steps per chunk
constexpr int R64_SPAN = 2 * R64_CHUNK;     // elements of K between two barriers: a chunk for each half
// a staged row takes eight elements more than a span: the sixteen lanes that read one
// step of sixteen rows then fall into different banks
constexpr int R64_STRIDE = R64_SPAN + 8;
constexpr int R64_AHEAD = 2 * R64_STEPS;    // weight fragments in flight a multiplying wave
constexpr int R64_MULTIPLIERS = 8;          // waves that multiply: four row groups x two halves of K
constexpr int R64_STAGERS = 8;              // waves that bring the rows
constexpr int R64_THREADS = (R64_MULTIPLIERS + R64_STAGERS) * 64;

enum { R64_STORE = 0, R64_SWIGLU = 1, R64_ADD = 2 };

extern __shared__ __attribute__((aligned(16))) unsigned char r64_lds[];

// two spans of rows; the sums of the waves of the second half pass through the same
// memory at the end (4 waves x 64 lanes x 4 MB values)
// (and, with the norm, the norm's weight: K values)
__host__ __device__ constexpr size_t r64_lds_bytes(int mb, int norm_k) {
  return (size_t)2 * mb * 16 * R64_STRIDE * sizeof(bf16_t) + 64 * sizeof(float) +
         (size_t)norm_k * sizeof(float);
}

template <int MB, int MODE, bool NORM>
__global__ void __launch_bounds__(R64_THREADS, 1)
gemm_bf16_rows64_kernel(const bf16_t* __restrict__ A, NormedRows64 normed,
                        const bf16_t* __restrict__ W, void* __restrict__ Cv, int M, int N, int K,
                        int kper) {
  constexpr int ROWS = MB * 16;
  bf16_t* ring = reinterpret_cast<bf16_t*>(r64_lds);
  float* ssw = reinterpret_cast<float*>(r64_lds + (size_t)2 * ROWS * R64_STRIDE * sizeof(bf16_t));
  [[maybe_unused]] float* nws = ssw + 64;                // the norm's weight [K]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kbase = blockIdx.y * kper;
  const int nspans = kper / R64_SPAN;                    // at least 2 (the launcher checks)
  auto slot = [&](int sp) { return ring + (size_t)(sp & 1) * ROWS * R64_STRIDE; };
  // Every workgroup walks its range of K from another span on, round: at any moment the
  // workgroups of a die then ask for different lines of the step's rows (which they all
  // read, and whose rows lie a power of two apart: the same span of every row sits in
  // the same few channels of the die's cache).
  // (workgroups are dealt to the eight dies in turn: those of one die are eight apart)
  const int rot = (int)((blockIdx.x / 8 + blockIdx.y) % (unsigned)nspans);
  auto phys = [&](int sp) { const int p = sp + rot; return p >= nspans ? p - nspans : p; };

  if (wave >= R64_MULTIPLIERS) {
    // ---------------------------------------------------------------- the rows
    // A wave takes PR rows; of a span, a lane takes four elements of each of the two
    // chunks of every row.  One span is in flight in registers while the one before it
    // is multiplied: requested in one interval, put into LDS in the next.
    constexpr int PR = 16 * MB / R64_STAGERS;            // rows of this wave
    const int row0 = (wave - R64_MULTIPLIERS) * PR;
    using Vec = typename std::conditional<NORM, f32x4_t, bf16x4_t>::type;
    // Two spans are in flight in registers where the registers allow it (DEEP): a span
    // requested at the start of one interval is put into LDS in the next but one, so a
    // request has two intervals to come back; otherwise one.
    constexpr bool DEEP = PR * (NORM ? 8 : 4) * 2 <= 64;
    constexpr int NB = DEEP ? 2 : 1;
    Vec buf[NB][PR][2];
    [[maybe_unused]] float ss[PR];
    unsigned base[PR];                                   // (the launcher checks that offsets fit)
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      // (a row beyond M repeats row M - 1: loaded and staged without conditions, never stored)
      int src = min(row0 + r, M - 1);
      if constexpr (NORM) {
        if (normed.rows) src = normed.rows[src];
        ss[r] = 0.f;
      }
      base[r] = (unsigned)src * (unsigned)K + kbase + lane * 4;
    }
    auto load = [&](auto b, int sp) {
#pragma unroll
      for (int r = 0; r < PR; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const size_t at = (size_t)base[r] + (size_t)phys(sp) * R64_SPAN + h * R64_CHUNK;
          if constexpr (NORM)
            buf[b][r][h] = *reinterpret_cast<const f32x4_t*>(normed.x + at);
          else
            buf[b][r][h] = *reinterpret_cast<const bf16x4_t*>(A + at);
        }
    };
    auto write = [&](auto b, int sp) {
      bf16_t* dst = slot(sp) + (size_t)row0 * R64_STRIDE + lane * 4;
#pragma unroll
      for (int r = 0; r < PR; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          bf16x4_t y;
          if constexpr (NORM) {
            const f32x4_t nw =
                *reinterpret_cast<const f32x4_t*>(nws + phys(sp) * R64_SPAN + h * R64_CHUNK + lane * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float a = buf[b][r][h][e];
              ss[r] += a * a;
              y[e] = (bf16_t)(a * nw[e]);
            }
          } else {
            y = buf[b][r][h];
          }
          *reinterpret_cast<bf16x4_t*>(dst + (size_t)r * R64_STRIDE + h * R64_CHUNK) = y;
        }
    };
    auto sums = [&]() {
      if constexpr (NORM) {
        // the rows' sums of squares, the lanes' shares added in a fixed order
#pragma unroll
        for (int r = 0; r < PR; ++r) {
          float v = ss[r];
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, ZA_WAVE);
          if (lane == 0) ssw[row0 + r] = v;
        }
      }
    };
    constexpr std::integral_constant<int, 0> B0{};
    constexpr std::integral_constant<int, NB - 1> B1{};
    auto stage_norm_weight = [&]() {
      // behind the first rows' requests: the norm's weight into LDS, by all staging waves
      if constexpr (NORM) {
        for (int k = (tid - R64_MULTIPLIERS * 64) * 4; k < K; k += R64_STAGERS * 64 * 4)
          *reinterpret_cast<f32x4_t*>(nws + k) = *reinterpret_cast<const f32x4_t*>(normed.weight + k);
        __syncthreads();
      }
    };
    if constexpr (DEEP) {
      // span s lives in buffer s & 1
      load(B0, 0);
      load(B1, 1);
      __builtin_amdgcn_sched_barrier(0);
      stage_norm_weight();
      write(B0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (2 < nspans) load(B0, 2);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();                                   // span 0 is staged
      // interval i (span i is multiplied): span i + 1 goes into LDS, span i + 3 is requested
      int i = 0;
      for (; i + 4 < nspans; i += 2) {
        write(B1, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        load(B1, i + 3);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        write(B0, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        load(B0, i + 4);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
      }
      for (; i < nspans; i += 2) {                       // the last spans, with conditions
        if (i + 1 < nspans) write(B1, i + 1);
        if (i + 3 < nspans) load(B1, i + 3);
        if (i + 1 >= nspans) sums();
        __syncthreads();
        if (i + 1 < nspans) {
          if (i + 2 < nspans) write(B0, i + 2);
          if (i + 4 < nspans) load(B0, i + 4);
          if (i + 2 >= nspans) sums();
          __syncthreads();
        }
      }
    } else {
      load(B0, 0);
      __builtin_amdgcn_sched_barrier(0);
      stage_norm_weight();
      write(B0, 0);
      __builtin_amdgcn_sched_barrier(0);
      load(B0, 1);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();                                   // span 0 is staged
      int i = 0;
      for (; i + 2 < nspans; ++i) {                      // while span i is multiplied
        write(B0, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        load(B0, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
      }
      write(B0, i + 1);                                  // i = nspans - 2: the last span
      __syncthreads();
      sums();
      __syncthreads();                                   // the last span is multiplied
    }
    __syncthreads();                                     // (the second half's sums pass through LDS)
    return;
  }

  // ------------------------------------------------------------------ the products
  // wave = 4 * half + group: the group's 16 weight rows, the half's chunk of every span
  const int group = wave & 3, half = wave >> 2;
  const int fr = lane & 15, fk = (lane >> 4) * 8, q = lane >> 4;
  int wrow;
  if constexpr (MODE == R64_SWIGLU) {
    const int j = min((int)blockIdx.x * 32 + group * 8 + (fr & 7), N - 1);
    wrow = fr < 8 ? j : N + j;
  } else {
    wrow = min((int)blockIdx.x * 64 + group * 16 + fr, N - 1);
  }
  const bf16_t* wp = W + (size_t)wrow * K + kbase + half * R64_CHUNK + fk;
  bf16x8_t fn[R64_AHEAD];
#pragma unroll
  for (int s = 0; s < R64_AHEAD; ++s)
    fn[s] = *reinterpret_cast<const bf16x8_t*>(wp + (size_t)phys(s / R64_STEPS) * R64_SPAN + (s % R64_STEPS) * 32);
  f32x4_t acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  if constexpr (NORM) __syncthreads();                   // (the staging waves hand each other the norm's weight)
  __syncthreads();                                       // span 0 is staged
  // One span: the wave's chunk of it, eight steps against the rows in LDS; `more`: the
  // fragment a step frees is requested anew at once, for the span after next.
  auto span = [&](int sp, auto parity, auto more) {
    const bf16_t* xs = slot(sp) + (size_t)fr * R64_STRIDE + half * R64_CHUNK + fk;
    const bf16_t* nxt = wp + (size_t)phys(sp + 2) * R64_SPAN;
    constexpr int at = decltype(parity)::value * R64_STEPS;
#pragma unroll
    for (int s = 0; s < R64_STEPS; ++s) {
      bf16x8_t xb[MB];
#pragma unroll
      for (int b = 0; b < MB; ++b)
        xb[b] = *reinterpret_cast<const bf16x8_t*>(xs + (size_t)b * 16 * R64_STRIDE + s * 32);
#pragma unroll
      for (int b = 0; b < MB; ++b)
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fn[at + s], xb[b], acc[b], 0, 0, 0);
      if constexpr (decltype(more)::value) {
        fn[at + s] = *reinterpret_cast<const bf16x8_t*>(nxt + s * 32);
        __builtin_amdgcn_sched_barrier(0);               // in this order: the compiler would bunch the loads
      }
    }
  };
  constexpr std::integral_constant<int, 0> P0{};
  constexpr std::integral_constant<int, 1> P1{};
  int i = 0;
  for (; i + 3 < nspans; i += 2) {
    span(i, P0, std::true_type{});
    __syncthreads();
    span(i + 1, P1, std::true_type{});
    __syncthreads();
  }
  // the last two or three spans: nothing left to request but, with three, the last
  if (i + 3 == nspans) {
    span(i, P0, std::true_type{});
    __syncthreads();
    span(i + 1, P1, std::false_type{});
    __syncthreads();
    span(i + 2, P0, std::false_type{});
    __syncthreads();
  } else {
    span(i, P0, std::false_type{});
    __syncthreads();
    span(i + 1, P1, std::false_type{});
    __syncthreads();
  }
  // the second half's sums meet the first half's: through LDS (the rows are done with)
  float* meet = reinterpret_cast<float*>(r64_lds);
  if (half == 1) {
#pragma unroll
    for (int b = 0; b < MB; ++b)
      *reinterpret_cast<f32x4_t*>(meet + ((size_t)(group * MB + b) * 64 + lane) * 4) = acc[b];
  }
  __syncthreads();
  if (half == 1) return;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const f32x4_t other = *reinterpret_cast<const f32x4_t*>(meet + ((size_t)(group * MB + b) * 64 + lane) * 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[b][r] += other[r];
  }

  // ------------------------------------------------------------------ what becomes of the sums
  // acc[b][r] is output (row m = 16 b + (lane & 15), weight row 4 q + r of the group's 16)
  if constexpr (MODE == R64_SWIGLU) {
    const int j0 = blockIdx.x * 32 + group * 8 + (q & 1) * 4;
    bf16_t* C = reinterpret_cast<bf16_t*>(Cv);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      float up[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) up[r] = __shfl_xor(acc[b][r], 32, ZA_WAVE);   // every lane takes part
      const int m = b * 16 + fr;
      if (q < 2 && m < M) {
        float scale = 1.f;
        if constexpr (NORM) scale = 1.0f / sqrtf(ssw[m] / (float)K + normed.eps);
        bf16x4_t y;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float gv = acc[b][r] * scale, uv = up[r] * scale;
          y[r] = (bf16_t)(gv * (1.0f / (1.0f + expf(-gv))) * uv);
        }
        if (j0 + 3 < N && N % 4 == 0) {
          *reinterpret_cast<bf16x4_t*>(C + (size_t)m * N + j0) = y;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (j0 + r < N) C[(size_t)m * N + j0 + r] = y[r];
        }
      }
    }
  } else {
    const int n0 = blockIdx.x * 64 + group * 16 + q * 4;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = b * 16 + fr;
      if (m >= M) continue;
      float scale = 1.f;
      if constexpr (NORM) scale = 1.0f / sqrtf(ssw[m] / (float)K + normed.eps);
      if constexpr (MODE == R64_ADD) {
        float* C = reinterpret_cast<float*>(Cv);
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n0 + r < N) unsafeAtomicAdd(C + (size_t)m * N + n0 + r, acc[b][r] * scale);
      } else {
        bf16_t* C = reinterpret_cast<bf16_t*>(Cv);
        bf16x4_t y;
#pragma unroll
        for (int r = 0; r < 4; ++r) y[r] = (bf16_t)(acc[b][r] * scale);
        if (n0 + 3 < N && N % 4 == 0) {
          *reinterpret_cast<bf16x4_t*>(C + (size_t)m * N + n0) = y;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n0 + r < N) C[(size_t)m * N + n0 + r] = y[r];
        }
      }
    }
  }
}

// A workgroup may ask for 64 KB of LDS at launch; a kernel that wants more is told so
// once.  The kernels are few: a short list remembers them.
int r64_allow_lds(const void* kernel, size_t bytes) {
  if (bytes <= 48 * 1024) return 0;
  static std::mutex guard;
  static std::vector<const void*> allowed;
  std::lock_guard<std::mutex> hold(guard);
  for (const void* k : allowed)
    if (k == kernel) return 0;
  const hipError_t rc =
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (rc != hipSuccess) {
    (void)hipGetLastError();
    return (int)rc;
  }
  allowed.push_back(kernel);
  return 0;
}

template <int MB, int MODE, bool NORM>
int r64_launch(const bf16_t* a, const NormedRows64& normed, const bf16_t* w, void* c, int M, int N,
               int K, int ksplit, hipStream_t stream) {
  auto kernel = gemm_bf16_rows64_kernel<MB, MODE, NORM>;
  const size_t lds = r64_lds_bytes(MB, NORM ? K : 0);
  const int rc = r64_allow_lds(reinterpret_cast<const void*>(kernel), lds);
  if (rc != 0) return rc;
  const int per_tile = MODE == R64_SWIGLU ? 32 : 64;
  dim3 grid((N + per_tile - 1) / per_tile, ksplit);
  hipLaunchKernelGGL(kernel, grid, dim3(R64_THREADS), lds, stream, a, normed, w, c, M, N, K, K / ksplit);
  return za_launch_status();
}

template <int MB>
int r64_dispatch(const bf16_t* a, const NormedRows64& normed, const bf16_t* w, void* c, int mode,
                 int M, int N, int K, int ksplit, hipStream_t stream) {
  const bool norm = normed.x != nullptr;
  if (mode == R64_STORE)
    return norm ? r64_launch<MB, R64_STORE, true>(a, normed, w, c, M, N, K, ksplit, stream)
                : r64_launch<MB, R64_STORE, false>(a, normed, w, c, M, N, K, ksplit, stream);
  if (mode == R64_SWIGLU)
    return norm ? r64_launch<MB, R64_SWIGLU, true>(a, normed, w, c, M, N, K, ksplit, stream)
                : r64_launch<MB, R64_SWIGLU, false>(a, normed, w, c, M, N, K, ksplit, stream);
  return r64_launch<MB, R64_ADD, false>(a, normed, w, c, M, N, K, ksplit, stream);
}

}  // namespace

// `a` [M, K] bfloat16, or (a null) `x` with `rows`, `norm_weight`, `eps`: rows of the
// 32-bit stream that the kernel normalises itself.  `w` [N, K] bfloat16 ([2 N, K] for
// mode 1).  `c`: mode 0 bfloat16 [M, N]; mode 1 bfloat16 [M, N]; mode 2 32-bit [M, N],
// added to.  K / ksplit must be a multiple of 512; ksplit > 1 only for mode 2; the norm
// only with modes 0 and 1.  Returns 0, ZA_ERR_ARG, ZA_ERR_UNSUPPORTED or a hipError_t.
extern "C" __attribute__((visibility("default")))
int za_gemm_bf16_rows64(const bf16_t* a, const float* x, const int* rows, const float* norm_weight,
                        float eps, const bf16_t* w, void* c, int mode, int M, int N, int K,
                        int ksplit, hipStream_t stream) {
  if (!w || !c || M < 1 || N < 1 || K < 1 || ksplit < 1 || mode < 0 || mode > 2) return ZA_ERR_ARG;
  if ((a == nullptr) == (x == nullptr)) return ZA_ERR_ARG;
  if (x && !norm_weight) return ZA_ERR_ARG;
  if (M > 64) return ZA_ERR_UNSUPPORTED;
  if (K % ksplit || (K / ksplit) % R64_SPAN || K / ksplit < 2 * R64_SPAN) return ZA_ERR_UNSUPPORTED;
  if (ksplit > 1 && mode != R64_ADD) return ZA_ERR_UNSUPPORTED;
  if (x && (mode == R64_ADD || K > 4096)) return ZA_ERR_UNSUPPORTED;   // (the norm's weight lies in LDS)
  if (ksplit > 65535) return ZA_ERR_UNSUPPORTED;
  // (the staging waves address the rows with 32-bit element offsets)
  if (!x && (unsigned long long)M * K >= (1ull << 31)) return ZA_ERR_UNSUPPORTED;
  const NormedRows64 normed = {x, rows, norm_weight, eps};
  switch ((M + 15) / 16) {
    case 1: return r64_dispatch<1>(a, normed, w, c, mode, M, N, K, ksplit, stream);
    case 2: return r64_dispatch<2>(a, normed, w, c, mode, M, N, K, ksplit, stream);
    case 3: return r64_dispatch<3>(a, normed, w, c, mode, M, N, K, ksplit, stream);
    default: return r64_dispatch<4>(a, normed, w, c, mode, M, N, K, ksplit, stream);
  }
}
