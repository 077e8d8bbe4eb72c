// C entry points of the CPU oracle (oracle/moe_oracle.cpp) that the C++ test
// programs link against: the checker, never the thing under test.
#pragma once
#include <cstddef>
extern "C" {
void oracle_forward(const float* tokens, const float* gate, const float* ffn1, const float* ffn2,
                    const float* bias, int T, int E, int H, int K, int I, float* out,
                    int* topk_idx, float* topk_w, int nthreads);
void oracle_reference_test_inputs(unsigned seed, float* tokens, size_t n_tokens, float* gate,
                                  size_t n_gate, float* ffn1, size_t n_ffn1, float* ffn2,
                                  size_t n_ffn2);
}
