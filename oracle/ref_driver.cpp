// TEST INFRASTRUCTURE ONLY. Thin extern "C" entry points over the reference's
// own header-only CPU MoE implementation, compiled from the headers where they
// lie in the reference checkout (-I<reference root>); nothing from the
// reference is copied into this repository. The resulting library goes to
// oracle/_ref/ and is used to validate the restatement in moe_oracle.cpp and
// to write the golden vectors under tests/golden/.
#include <cstddef>
#include <cstring>
#include <vector>

#include "test/singleGPU/cpp/moe/reference/refFullMoe.h"

extern "C" {

void ref_gemm(const float* a, const float* b, int m, int n, int k, float* c) {
  const std::vector<float> r = test::refGemm(a, b, m, n, k);
  std::memcpy(c, r.data(), r.size() * sizeof(float));
}

void ref_topk(const float* in, int rows, int cols, int topk, float* vals,
              int* idx) {
  test::refTopK8PerRow(in, rows, cols, vals, idx, topk);
}

void ref_softmax_rows(float* data, int rows, int cols) {
  test::refSoftmaxRowOnlineInplace(data, rows, cols);
}

void ref_moe_gate(const float* tokens, const float* gate, int T, int E, int H,
                  int K, float* topk_w, int* topk_idx) {
  const test::MoeGateOutput g = test::refMoeGate(tokens, gate, T, E, H, K);
  std::memcpy(topk_w, g.topkVals.data(), g.topkVals.size() * sizeof(float));
  std::memcpy(topk_idx, g.topkIdx.data(), g.topkIdx.size() * sizeof(int));
}

void ref_expert_ffn1(const float* tokens, const float* w13, int T, int H, int I,
                     float* out) {
  const std::vector<float> r = test::refExpertFFN1(tokens, w13, T, H, I);
  std::memcpy(out, r.data(), r.size() * sizeof(float));
}

void ref_full_moe(const float* tokens, const float* gate, const float* ffn1,
                  const float* ffn2, int T, int E, int H, int K, int I,
                  float* out) {
  const std::vector<float> r =
      test::refFullMoe(tokens, gate, ffn1, ffn2, T, E, H, K, I);
  std::memcpy(out, r.data(), r.size() * sizeof(float));
}

}  // extern "C"
