// TEST INFRASTRUCTURE ONLY. This file is the CPU oracle for the fused MoE
// layer: a restatement of the reference's CPU MoE implementation with runtime
// shapes. It is the checker for the HIP path and the "cpu_baseline" leg of the
// benchmark; nothing in the product library links, loads or calls it.
//
// Each function names the reference file:line whose arithmetic and ordering it
// follows (paths relative to the reference checkout):
//   test/singleGPU/cpp/moe/reference/refGemm.h:11-30      sequential-k GEMM
//   test/singleGPU/cpp/moe/reference/refTopk.h:17-68      insertion top-k
//   test/singleGPU/cpp/moe/reference/refSoftmax.h:15-53   online softmax (double)
//   test/singleGPU/cpp/moe/reference/refMoeGate.h:16-33   router = gemm+topk+softmax
//   test/singleGPU/cpp/moe/reference/refExpertFFN1.h:12-65 SiLU(a)*b
//   test/singleGPU/cpp/moe/reference/refFullMoe.h:9-70    whole layer
//
// Pinning status (what checks each function, see tests/test_oracle_*.py):
//   oracle_logits      : golden vectors from the compiled reference headers,
//                        float64 numpy matmul, exact integer-valued cases
//   oracle_topk        : golden vectors, stable argsort closed form, tie fixtures
//   oracle_softmax_topk: golden vectors, float64 softmax, sum-to-one invariant
//   oracle_gate        : golden vectors (composition of the three above)
//   oracle_forward     : golden vectors, dense float64 einsum restatement
//   oracle_permute     : NOT in the reference (it has no permutation stage).
//                        Pinned by the closed form "stable sort of (token,slot)
//                        assignments by expert id" and by brute force; parity
//                        with the reference itself is unpinned by construction.
//
// Additions that are not in the reference and reduce to it when unused:
//   * optional router bias added to the logits after the GEMM and before top-k
//   * token-sharded threads (tokens are independent, refFullMoe.h:32), results
//     are identical for any thread count
//
// Build: g++ -O2 -ffp-contract=off (no FMA contraction, no -march=native, no
// -ffast-math) so the float arithmetic is the plain IEEE sequence.

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

namespace {

// refGemm.h:16-27 — one output element: acc starts at 0 and adds the products
// a[k]*b[k] one by one, k ascending, all in float.
inline float dot_seq(const float* a, const float* b, int K) {
  float acc = 0.0f;
  for (int k = 0; k < K; ++k) acc += a[k] * b[k];
  return acc;
}

// refTopk.h:25-59 — scan the columns left to right, keep a descending list of
// TOPK values; a value is inserted before the first kept value it is strictly
// greater than, so equal values keep ascending column order and NaN never
// enters. Unfilled slots keep lowest()/-1 (refTopk.h:22,30-33).
inline void topk_row(const float* row, int cols, int topk, float* vals,
                     int* idx) {
  const float lowest = std::numeric_limits<float>::lowest();
  for (int t = 0; t < topk; ++t) {
    vals[t] = lowest;
    idx[t] = -1;
  }
  for (int c = 0; c < cols; ++c) {
    const float v = row[c];
    int pos = topk;
    for (int t = 0; t < topk; ++t) {
      if (v > vals[t]) {
        pos = t;
        break;
      }
    }
    if (pos == topk) continue;
    for (int t = topk - 1; t > pos; --t) {
      vals[t] = vals[t - 1];
      idx[t] = idx[t - 1];
    }
    vals[pos] = v;
    idx[pos] = c;
  }
}

// refSoftmax.h:19-52 — running max and rescaled sum in double, then
// exp(x-max)/sum cast back to float; a non-positive sum yields the uniform row.
inline void softmax_row(float* row, int cols) {
  if (cols == 0) return;
  double maxv = static_cast<double>(row[0]);
  double sum = 1.0;
  for (int j = 1; j < cols; ++j) {
    const double x = static_cast<double>(row[j]);
    if (x > maxv) {
      sum = sum * std::exp(maxv - x) + 1.0;
      maxv = x;
    } else {
      sum += std::exp(x - maxv);
    }
  }
  if (sum <= 0.0) {
    const float inv = static_cast<float>(1.0 / static_cast<double>(cols));
    for (int j = 0; j < cols; ++j) row[j] = inv;
  } else {
    for (int j = 0; j < cols; ++j) {
      const double e = std::exp(static_cast<double>(row[j]) - maxv);
      row[j] = static_cast<float>(e / sum);
    }
  }
}

// refExpertFFN1.h:12-21 — sign-split sigmoid in float.
inline float sigmoid_split(float x) {
  if (x >= 0.0f) {
    const float e = std::exp(-x);
    return 1.0f / (1.0f + e);
  }
  const float e = std::exp(x);
  return e / (1.0f + e);
}

struct Shape {
  int T, E, H, K, I;
};

void gate_range(const float* tokens, const float* gate, const float* bias,
                const Shape& s, int t0, int t1, float* logits_out,
                int* topk_idx, float* topk_w) {
  std::vector<float> row(static_cast<size_t>(s.E));
  for (int t = t0; t < t1; ++t) {
    const float* x = tokens + static_cast<size_t>(t) * s.H;
    for (int e = 0; e < s.E; ++e) {
      float v = dot_seq(x, gate + static_cast<size_t>(e) * s.H, s.H);
      if (bias) v = v + bias[e];
      row[e] = v;
    }
    if (logits_out)
      std::memcpy(logits_out + static_cast<size_t>(t) * s.E, row.data(),
                  sizeof(float) * s.E);
    float* w = topk_w + static_cast<size_t>(t) * s.K;
    int* ix = topk_idx + static_cast<size_t>(t) * s.K;
    topk_row(row.data(), s.E, s.K, w, ix);
    softmax_row(w, s.K);  // refMoeGate.h:30: softmax over the k winning logits
  }
}

// refFullMoe.h:32-66 for tokens [t0,t1): per slot in descending-weight order,
// FFN1 (refExpertFFN1.h:51-65) then FFN2 (refGemm) then out += y*w.
void experts_range(const float* tokens, const float* ffn1, const float* ffn2,
                   const Shape& s, const int* topk_idx, const float* topk_w,
                   int t0, int t1, float* out) {
  std::vector<float> gu(static_cast<size_t>(2) * s.I);
  std::vector<float> h(static_cast<size_t>(s.I));
  for (int t = t0; t < t1; ++t) {
    const float* x = tokens + static_cast<size_t>(t) * s.H;
    float* o = out + static_cast<size_t>(t) * s.H;
    for (int d = 0; d < s.H; ++d) o[d] = 0.0f;
    for (int slot = 0; slot < s.K; ++slot) {
      const int e = topk_idx[static_cast<size_t>(t) * s.K + slot];
      const float w = topk_w[static_cast<size_t>(t) * s.K + slot];
      if (e < 0 || e >= s.E || ffn1 == nullptr) continue;  // refFullMoe.h:40-43
      const float* w13 = ffn1 + static_cast<size_t>(e) * 2 * s.I * s.H;
      const float* w2 = ffn2 + static_cast<size_t>(e) * s.H * s.I;
      for (int n = 0; n < 2 * s.I; ++n)
        gu[n] = dot_seq(x, w13 + static_cast<size_t>(n) * s.H, s.H);
      for (int c = 0; c < s.I; ++c) {
        const float a = gu[c];
        const float b = gu[s.I + c];
        const float sg = sigmoid_split(a);
        h[c] = a * sg * b;  // refExpertFFN1.h:45
      }
      for (int d = 0; d < s.H; ++d) {
        const float y = dot_seq(h.data(), w2 + static_cast<size_t>(d) * s.I, s.I);
        o[d] += y * w;  // refFullMoe.h:62-65
      }
    }
  }
}

template <typename F>
void shard_tokens(int T, int nthreads, F&& body) {
  if (nthreads <= 1 || T <= 1) {
    body(0, T);
    return;
  }
  if (nthreads > T) nthreads = T;
  std::vector<std::thread> pool;
  const int base = T / nthreads, rem = T % nthreads;
  int t0 = 0;
  for (int i = 0; i < nthreads; ++i) {
    const int n = base + (i < rem ? 1 : 0);
    pool.emplace_back([=, &body] { body(t0, t0 + n); });
    t0 += n;
  }
  for (auto& th : pool) th.join();
}

}  // namespace

extern "C" {

// logits[T,E] = tokens[T,H] . gate[E,H]^T (+ bias[E]).
void oracle_logits(const float* tokens, const float* gate, const float* bias,
                   int T, int E, int H, float* logits, int nthreads) {
  shard_tokens(T, nthreads, [&](int t0, int t1) {
    for (int t = t0; t < t1; ++t)
      for (int e = 0; e < E; ++e) {
        float v = dot_seq(tokens + static_cast<size_t>(t) * H,
                          gate + static_cast<size_t>(e) * H, H);
        if (bias) v = v + bias[e];
        logits[static_cast<size_t>(t) * E + e] = v;
      }
  });
}

// Row-wise top-k of a [rows, cols] matrix: descending values, ties by
// ascending column.
void oracle_topk(const float* input, int rows, int cols, int topk, float* vals,
                 int* idx) {
  for (int r = 0; r < rows; ++r)
    topk_row(input + static_cast<size_t>(r) * cols, cols, topk,
             vals + static_cast<size_t>(r) * topk,
             idx + static_cast<size_t>(r) * topk);
}

// In-place row softmax of a [rows, cols] matrix.
void oracle_softmax_rows(float* data, int rows, int cols) {
  for (int r = 0; r < rows; ++r)
    softmax_row(data + static_cast<size_t>(r) * cols, cols);
}

// Router: logits (+bias) -> top-k indices -> softmax over the winners.
void oracle_gate(const float* tokens, const float* gate, const float* bias,
                 int T, int E, int H, int K, float* logits /*nullable*/,
                 int* topk_idx, float* topk_w, int nthreads) {
  const Shape s{T, E, H, K, 0};
  shard_tokens(T, nthreads, [&](int t0, int t1) {
    gate_range(tokens, gate, bias, s, t0, t1, logits, topk_idx, topk_w);
  });
}

// Per-expert token permutation: stable counting sort of the assignments
// (token t, slot s), visited in ascending t*K+s, by expert id. counts[E],
// offsets[E+1] (exclusive scan), perm[offsets[e]+j] = t*K+s. Assignments with
// an index outside [0,E) are dropped. Returns the number of rows placed.
int oracle_permute(const int* topk_idx, int T, int E, int K, int* counts,
                   int* offsets, int* perm) {
  for (int e = 0; e < E; ++e) counts[e] = 0;
  for (int i = 0; i < T * K; ++i) {
    const int e = topk_idx[i];
    if (e >= 0 && e < E) counts[e]++;
  }
  offsets[0] = 0;
  for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
  std::vector<int> fill(offsets, offsets + E);
  for (int i = 0; i < T * K; ++i) {
    const int e = topk_idx[i];
    if (e >= 0 && e < E) perm[fill[e]++] = i;
  }
  return offsets[E];
}

// Whole layer. out[T,H]; topk_idx/topk_w [T,K] are outputs (nullable).
void oracle_forward(const float* tokens, const float* gate, const float* ffn1,
                    const float* ffn2, const float* bias, int T, int E, int H,
                    int K, int I, float* out, int* topk_idx, float* topk_w,
                    int nthreads) {
  const Shape s{T, E, H, K, I};
  std::vector<int> idx_local;
  std::vector<float> w_local;
  if (!topk_idx) {
    idx_local.resize(static_cast<size_t>(T) * K);
    topk_idx = idx_local.data();
  }
  if (!topk_w) {
    w_local.resize(static_cast<size_t>(T) * K);
    topk_w = w_local.data();
  }
  shard_tokens(T, nthreads, [&](int t0, int t1) {
    gate_range(tokens, gate, bias, s, t0, t1, nullptr, topk_idx, topk_w);
    experts_range(tokens, ffn1, ffn2, s, topk_idx, topk_w, t0, t1, out);
  });
}

// Expert stage only, for a routing given by the caller (used to check the
// expert GEMMs independently of the router).
void oracle_experts(const float* tokens, const float* ffn1, const float* ffn2,
                    int T, int E, int H, int K, int I, const int* topk_idx,
                    const float* topk_w, float* out, int nthreads) {
  const Shape s{T, E, H, K, I};
  shard_tokens(T, nthreads, [&](int t0, int t1) {
    experts_range(tokens, ffn1, ffn2, s, topk_idx, topk_w, t0, t1, out);
  });
}

// The input generator of the reference's own tests: srand(7907) once, then
// low + (rand()/RAND_MAX)*(high-low) in float, drawn in the order tokens,
// gate, ffn1, ffn2 (test/common/utils.h:9,62-87; test/common/moeTools.h:45-69:
// tokens in [-1,1], every weight in [-0.1,0.1]). glibc rand() is a process
// global: call this from one thread only.
void oracle_reference_test_inputs(unsigned seed, float* tokens, size_t n_tokens,
                                  float* gate, size_t n_gate, float* ffn1,
                                  size_t n_ffn1, float* ffn2, size_t n_ffn2) {
  srand(seed);
  auto draw = [](float lo, float hi) {
    const float u = static_cast<float>(rand()) / static_cast<float>(RAND_MAX);
    return lo + static_cast<float>(u * static_cast<float>(hi - lo));
  };
  for (size_t i = 0; i < n_tokens; ++i) tokens[i] = draw(-1.0f, 1.0f);
  for (size_t i = 0; i < n_gate; ++i) gate[i] = draw(-0.1f, 0.1f);
  for (size_t i = 0; i < n_ffn1; ++i) ffn1[i] = draw(-0.1f, 0.1f);
  for (size_t i = 0; i < n_ffn2; ++i) ffn2[i] = draw(-0.1f, 0.1f);
}

}  // extern "C"
