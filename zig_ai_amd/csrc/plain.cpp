// Plain statements, in C++ on host memory, of what each kernel under this folder
// computes: one function per kernel, with the kernel's own operands (the packed
// step, the paged cache with its block table, the state slots), everything in
// 32-bit floats with sums in double precision, one loop nest each and no attempt
// at speed.  They exist to check the kernels (and the layouts the kernels assume)
// from a second side; the engine never calls them.
//
// Formulas, from the reference:
//   RMSNorm                 /root/reference/src/transformer/norm.zig:6-33
//   rotary encoding         /root/reference/src/transformer/rope.zig:23-57,
//                           /root/reference/src/cuda/layer_kernels.cu:353-365 (half pairing)
//   per-head q/k norm       /root/reference/src/transformer/hybrid_attn.zig:371-382
//   attention               /root/reference/src/transformer/hybrid_attn.zig:553-608
//   query head -> kv head   /root/reference/src/transformer/gqa.zig:87-106
//   SwiGLU                  /root/reference/src/transformer/ffn.zig:19-33
//   convolution with state  /root/reference/src/transformer/short_conv.zig:188-225
//   sampler                 /root/reference/src/transformer/pipeline.zig:25-181
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#include <algorithm>
#include <vector>

#define ZA_API extern "C" __attribute__((visibility("default")))

namespace {
constexpr int OK = 0;
constexpr int BAD_ARGUMENT = 1;
}  // namespace

// residual [T, H] (may be null: then the sum is `delta` alone) += sum over the P
// stacked terms of delta [P, T, H] (may be null); out = RMSNorm(residual) * w.
ZA_API int za_plain_add_rmsnorm(float* residual, const float* delta, int P, const float* w,
                                float* out, int T, int H, float eps) {
  if (T < 0 || H <= 0 || (!residual && !delta)) return BAD_ARGUMENT;
  std::vector<float> row(H);
  for (int t = 0; t < T; ++t) {
    for (int i = 0; i < H; ++i) {
      float v = residual ? residual[(size_t)t * H + i] : 0.0f;
      if (delta)
        for (int p = 0; p < P; ++p) v += delta[((size_t)p * T + t) * H + i];
      row[i] = v;
      if (residual) residual[(size_t)t * H + i] = v;
    }
    double ss = 0.0;
    for (int i = 0; i < H; ++i) ss += (double)row[i] * row[i];
    const double scale = 1.0 / sqrt(ss / H + (double)eps);
    for (int i = 0; i < H; ++i) out[(size_t)t * H + i] = (float)(row[i] * scale * w[i]);
  }
  return OK;
}

// out[t] = table[tokens[t]]; a token outside the table is an error.
ZA_API int za_plain_embed(const int* tokens, const float* table, float* out, int T, int H,
                          int vocab) {
  for (int t = 0; t < T; ++t) {
    if (tokens[t] < 0 || tokens[t] >= vocab) return BAD_ARGUMENT;
    for (int i = 0; i < H; ++i) out[(size_t)t * H + i] = table[(size_t)tokens[t] * H + i];
  }
  return OK;
}

// y [M, N] = x [M, K] . w [N, K]^T (+ bias [N])
ZA_API int za_plain_linear(const float* x, const float* w, const float* bias, float* y, int M,
                           int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double s = bias ? (double)bias[n] : 0.0;
      for (int k = 0; k < K; ++k) s += (double)x[(size_t)m * K + k] * w[(size_t)n * K + k];
      y[(size_t)m * N + n] = (float)s;
    }
  return OK;
}

// gate_up [T, 2I] = [gate | up];  out [T, I] = gate / (1 + exp(-gate)) * up
ZA_API int za_plain_swiglu(const float* gate_up, float* out, int T, int I) {
  for (int t = 0; t < T; ++t)
    for (int i = 0; i < I; ++i) {
      const double g = gate_up[(size_t)t * 2 * I + i], u = gate_up[(size_t)t * 2 * I + I + i];
      out[(size_t)t * I + i] = (float)(g / (1.0 + exp(-g)) * u);
    }
  return OK;
}

// qkv [T, (nh + 2 nkv) * d], heads in the order q..., k..., v...  The queries come
// back normalised and rotated in q_out [T, nh, d]; keys (normalised, rotated) and
// values (as they are) go to the cache [pages, 2, nkv, page_size * d] at
// slot = page * page_size + offset: a key as [offset][d], a value as [d][offset].
ZA_API int za_plain_qk_norm_rope_kv_write(const float* qkv, const int* positions,
                                          const int* slots, const float* q_norm_w,
                                          const float* k_norm_w, const float* inv_freq,
                                          float* q_out, float* kv_cache, int T, int nh, int nkv,
                                          int d, int rotary_dim, int adjacent_pairs, float eps,
                                          int page_size, int write_kv) {
  if (rotary_dim % 2 || rotary_dim > d) return BAD_ARGUMENT;
  const int total = nh + 2 * nkv;
  std::vector<double> v(d), r(d);
  for (int t = 0; t < T; ++t)
    for (int head = 0; head < total; ++head) {
      const bool is_q = head < nh, is_k = !is_q && head < nh + nkv;
      const float* src = qkv + ((size_t)t * total + head) * d;
      for (int i = 0; i < d; ++i) v[i] = src[i];
      const float* nw = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
      if (nw) {
        double ss = 0.0;
        for (int i = 0; i < d; ++i) ss += v[i] * v[i];
        const double scale = 1.0 / sqrt(ss / d + (double)eps);
        for (int i = 0; i < d; ++i) v[i] = v[i] * scale * nw[i];
      }
      if ((is_q || is_k) && rotary_dim > 0) {
        r = v;
        const int half = rotary_dim / 2;
        for (int p = 0; p < half; ++p) {
          const int a = adjacent_pairs ? 2 * p : p, b = adjacent_pairs ? 2 * p + 1 : p + half;
          // the angle in 32-bit, as the model defines it: position * inv_freq
          const double angle = (double)((float)positions[t] * inv_freq[p]);
          r[a] = v[a] * cos(angle) - v[b] * sin(angle);
          r[b] = v[a] * sin(angle) + v[b] * cos(angle);
        }
        v = r;
      }
      if (is_q) {
        for (int i = 0; i < d; ++i) q_out[((size_t)t * nh + head) * d + i] = (float)v[i];
      } else if (write_kv) {
        const int kv = is_k ? head - nh : head - nh - nkv;
        const int page = slots[t] / page_size, off = slots[t] % page_size;
        float* base = kv_cache + (((size_t)page * 2 + (is_k ? 0 : 1)) * nkv + kv) * page_size * d;
        for (int i = 0; i < d; ++i) {
          if (is_k) base[(size_t)off * d + i] = (float)v[i];
          else base[(size_t)i * page_size + off] = (float)v[i];
        }
      }
    }
  return OK;
}

// Token t of request token_seq[t] at position positions[t] attends the keys at
// positions max(0, pos - window + 1) .. pos of its own request (window 0: all of
// them), found through block_table [requests, table_width]; softmax in two passes.
ZA_API int za_plain_paged_attention(const float* q, float* out, const float* kv_cache,
                                    const int* block_table, int table_width,
                                    const int* positions, const int* token_seq, int T, int nh,
                                    int nkv, int d, int page_size, float scale, int window) {
  if (nkv <= 0 || nh % nkv) return BAD_ARGUMENT;
  const int group = nh / nkv;
  std::vector<double> score, acc(d);
  for (int t = 0; t < T; ++t) {
    const int pos = positions[t];
    const int first = window > 0 ? std::max(0, pos - window + 1) : 0;
    if ((pos / page_size) >= table_width) return BAD_ARGUMENT;
    const int* table = block_table + (size_t)token_seq[t] * table_width;
    for (int h = 0; h < nh; ++h) {
      const int kv = h / group;
      const float* qv = q + ((size_t)t * nh + h) * d;
      score.assign(pos - first + 1, 0.0);
      double top = -INFINITY;
      for (int j = first; j <= pos; ++j) {
        const float* kp = kv_cache + (((size_t)table[j / page_size] * 2 + 0) * nkv + kv) * page_size * d +
                          (size_t)(j % page_size) * d;
        double s = 0.0;
        for (int i = 0; i < d; ++i) s += (double)qv[i] * kp[i];
        score[j - first] = s * scale;
        top = std::max(top, score[j - first]);
      }
      double sum = 0.0;
      for (double& s : score) { s = exp(s - top); sum += s; }
      std::fill(acc.begin(), acc.end(), 0.0);
      for (int j = first; j <= pos; ++j) {
        const float* vp = kv_cache + (((size_t)table[j / page_size] * 2 + 1) * nkv + kv) * page_size * d +
                          (j % page_size);
        for (int i = 0; i < d; ++i) acc[i] += score[j - first] * vp[(size_t)i * page_size];
      }
      for (int i = 0; i < d; ++i) out[((size_t)t * nh + h) * d + i] = (float)(acc[i] / sum);
    }
  }
  return OK;
}

// z [T, 3 width] = [B | C | X]; w [width, L] as a checkpoint holds the filter (tap
// L-1 multiplies the present input); state [slots, width, L]: the last L inputs
// u = B * X of the request, oldest first.  Request s owns tokens seq_start[s] ..
// seq_start[s+1]-1 and slot slot_id[s].  y [T, width] = C * (bias + sum_j w[ch][j] *
// u[t - (L-1) + j]); the state afterwards holds the last L inputs again.
ZA_API int za_plain_short_conv(const float* z, const float* w, const float* bias, float* state,
                               const int* seq_start, const int* slot_id, float* y, int n_seqs,
                               int width, int L) {
  if (L < 1) return BAD_ARGUMENT;
  for (int s = 0; s < n_seqs; ++s) {
    const int t0 = seq_start[s], n = seq_start[s + 1] - t0;
    float* st = state + (size_t)slot_id[s] * width * L;
    for (int ch = 0; ch < width; ++ch) {
      std::vector<double> u(L + n);           // u[L + i] is the input of token t0 + i
      for (int j = 0; j < L; ++j) u[j] = st[(size_t)ch * L + j];
      for (int i = 0; i < n; ++i) {
        const float* row = z + (size_t)(t0 + i) * 3 * width;
        u[L + i] = (double)row[ch] * row[2 * width + ch];
      }
      for (int i = 0; i < n; ++i) {
        double c = bias ? (double)bias[ch] : 0.0;
        for (int j = 0; j < L; ++j) c += (double)w[(size_t)ch * L + j] * u[L + i - (L - 1) + j];
        y[(size_t)(t0 + i) * width + ch] = (float)(z[(size_t)(t0 + i) * 3 * width + width + ch] * c);
      }
      for (int j = 0; j < L; ++j) st[(size_t)ch * L + j] = (float)u[n + j];
    }
  }
  return OK;
}

// First index of each row's maximum.
ZA_API int za_plain_argmax(const float* logits, int rows, int vocab, int* out) {
  for (int r = 0; r < rows; ++r) {
    const float* row = logits + (size_t)r * vocab;
    int best = 0;
    for (int i = 1; i < vocab; ++i)
      if (row[i] > row[best]) best = i;
    out[r] = best;
  }
  return OK;
}

// Positive logits of the listed (row, token) pairs are divided by the pair's
// factor, negative ones multiplied.
ZA_API int za_plain_repetition_penalty(float* logits, int vocab, const int* rows,
                                       const int* tokens, const float* factors, int n) {
  for (int i = 0; i < n; ++i) {
    if (tokens[i] < 0 || tokens[i] >= vocab) return BAD_ARGUMENT;
    float& v = logits[(size_t)rows[i] * vocab + tokens[i]];
    v = v > 0.0f ? v / factors[i] : v * factors[i];
  }
  return OK;
}

// One row: v = logit / temperature; keep[i] says whether token i survives top-k
// (v >= the k-th largest; k <= 0 or k >= vocab: all) and then top-p (the largest
// values, taken in descending order until their share of the kept probability
// reaches p, and every value equal to the last one taken; p >= 1: all); weight[i]
// = exp(v_i - max) for kept tokens, 0 otherwise.
ZA_API int za_plain_sample_weights(const float* logits, int vocab, float temperature, int top_k,
                                   float top_p, double* weight, unsigned char* keep) {
  if (temperature <= 0.0f || vocab <= 0) return BAD_ARGUMENT;
  std::vector<double> v(vocab);
  for (int i = 0; i < vocab; ++i) v[i] = (double)logits[i] / (double)temperature;
  std::vector<double> sorted(v);
  std::sort(sorted.begin(), sorted.end(), [](double a, double b) { return a > b; });
  double floor_value = -INFINITY;
  if (top_k > 0 && top_k < vocab) floor_value = sorted[top_k - 1];
  const double top = sorted[0];
  if (top_p < 1.0f) {
    double total = 0.0;
    for (int i = 0; i < vocab && sorted[i] >= floor_value; ++i) total += exp(sorted[i] - top);
    double run = 0.0;
    for (int i = 0; i < vocab && sorted[i] >= floor_value; ++i) {
      run += exp(sorted[i] - top);
      if (run >= (double)top_p * total) {
        floor_value = sorted[i];
        break;
      }
    }
  }
  for (int i = 0; i < vocab; ++i) {
    keep[i] = v[i] >= floor_value ? 1 : 0;
    weight[i] = keep[i] ? exp(v[i] - top) : 0.0;
  }
  return OK;
}

// One token per row: the first maximum where temperature <= 0, else the first kept
// index i, in index order, whose running weight reaches uniform * (sum of weights);
// the last kept index if rounding leaves none.
ZA_API int za_plain_sample(const float* logits, int rows, int vocab, const float* temperature,
                           const int* top_k, const float* top_p, const float* uniform, int* out) {
  std::vector<double> weight(vocab);
  std::vector<unsigned char> keep(vocab);
  for (int r = 0; r < rows; ++r) {
    const float* row = logits + (size_t)r * vocab;
    if (temperature[r] <= 0.0f) {
      za_plain_argmax(row, 1, vocab, out + r);
      continue;
    }
    const int rc = za_plain_sample_weights(row, vocab, temperature[r], top_k[r], top_p[r],
                                           weight.data(), keep.data());
    if (rc != OK) return rc;
    double total = 0.0;
    for (int i = 0; i < vocab; ++i) total += weight[i];
    const double target = (double)uniform[r] * total;
    double run = 0.0;
    int chosen = -1, last = 0;
    for (int i = 0; i < vocab && chosen < 0; ++i) {
      if (!keep[i] || weight[i] <= 0.0) continue;
      last = i;
      run += weight[i];
      if (run >= target) chosen = i;
    }
    out[r] = chosen >= 0 ? chosen : last;
  }
  return OK;
}
