// The reference's launcher benchmark
// (test/singleGPU/cpp/benchmarks/moeKernelBenchmark.cpp:23-90: 10 warm-up and
// 10 timed launches between two events, T = 1, 16, 32) re-targeted at this
// library and widened: the same float sweep through CreateLauncher, extended to
// the batch sizes the reference cannot hold, then the bf16 30B shape through
// CreateLauncherEx at the decode and prefill batch sizes. Weights and tokens are
// initialised (uniform, the reference generator's ranges) so that routing
// spreads over the experts as in a real layer.
#include <cstdint>
#include <cstdio>
#include <vector>

#include "include/iMoeKernelLauncher.h"
#include "tests/cpp/mini_test.h"

namespace {

constexpr int EXPERTS_NUM = 128, HIDDEN_SIZE = 2048, EXPERT_INTERMEDIATE_SIZE = 768, TOPK = 8;

struct Lcg {
  uint64_t s;
  float next(float lo, float hi) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return lo + (hi - lo) * static_cast<float>((s >> 40) * (1.0 / 16777216.0));
  }
};

uint16_t ToBf16(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// n values in [lo, hi] on the device, float or bf16
void* RandomDevice(size_t n, float lo, float hi, bool bf16, uint64_t seed) {
  Lcg g{seed};
  void* d = nullptr;
  if (bf16) {
    std::vector<uint16_t> h(n);
    for (auto& v : h) v = ToBf16(g.next(lo, hi));
    if (hipMalloc(&d, n * 2) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), n * 2, hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  } else {
    std::vector<float> h(n);
    for (auto& v : h) v = g.next(lo, hi);
    if (hipMalloc(&d, n * 4) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), n * 4, hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  }
  return d;
}

// test/singleGPU/cpp/benchmarks/benchmarkUtils.h:26-52
template <typename F>
float Benchmark(int warmup, int iters, hipStream_t stream, F&& f) {
  for (int i = 0; i < warmup; ++i) f();
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  hipEventRecord(a, stream);
  for (int i = 0; i < iters; ++i) f();
  hipEventRecord(b, stream);
  hipEventSynchronize(b);
  float ms = 0.f;
  hipEventElapsedTime(&ms, a, b);
  hipEventDestroy(a);
  hipEventDestroy(b);
  return ms / iters;
}

struct Weights {
  void *gate = nullptr, *ffn1 = nullptr, *ffn2 = nullptr;
  bool bf16 = false;
};

Weights MakeWeights(bool bf16) {
  Weights w;
  w.bf16 = bf16;
  w.gate = RandomDevice(static_cast<size_t>(EXPERTS_NUM) * HIDDEN_SIZE, -0.1f, 0.1f, bf16, 1);
  w.ffn1 = RandomDevice(static_cast<size_t>(EXPERTS_NUM) * 2 * EXPERT_INTERMEDIATE_SIZE * HIDDEN_SIZE,
                        -0.1f, 0.1f, bf16, 2);
  w.ffn2 = RandomDevice(static_cast<size_t>(EXPERTS_NUM) * HIDDEN_SIZE * EXPERT_INTERMEDIATE_SIZE,
                        -0.1f, 0.1f, bf16, 3);
  return w;
}

void PerformBenchmark(const Weights& w, int numTokens, bool& mini_ok) {
  hipStream_t stream = 0;
  const size_t elems = static_cast<size_t>(numTokens) * HIDDEN_SIZE;
  void* tokens_device = RandomDevice(elems, -1.0f, 1.0f, w.bf16, 4);
  void* finalOutput_device = nullptr;
  ASSERT_TRUE(tokens_device != nullptr);
  HIP_ERROR_ASSERT(hipMalloc(&finalOutput_device, elems * (w.bf16 ? 2 : 4)));
  const moe::DistributedUniqueId duid = GetDistributedUniqueId(/*empty=*/true);
  moe::IMoeKernelLauncher* launcher = nullptr;
  if (!w.bf16) {
    HIP_ERROR_ASSERT(CreateLauncher(&launcher, w.gate, w.ffn1, w.ffn2, numTokens, stream, duid, 0, 1));
  } else {
    FlashMoeLayerDesc d = {};
    d.experts = EXPERTS_NUM;
    d.hidden = HIDDEN_SIZE;
    d.intermediate = EXPERT_INTERMEDIATE_SIZE;
    d.top_k = TOPK;
    d.dtype = FLASH_MOE_BF16;
    d.max_tokens = numTokens;
    d.sched = FLASH_MOE_SCHED_AUTO;
    d.gate_weights = w.gate;
    d.ffn1_weights = w.ffn1;
    d.ffn2_weights = w.ffn2;
    HIP_ERROR_ASSERT(CreateLauncherEx(&launcher, &d, stream));
  }
  const float avg_ms = Benchmark(10, 10, stream, [&] {
    launcher->Launch(tokens_device, finalOutput_device, numTokens, stream);
  });
  HIP_ERROR_ASSERT(hipDeviceSynchronize());
  HIP_ERROR_ASSERT(hipGetLastError());
  unsigned bits = 0;
  unsigned launches = 0;
  ASSERT_EQ(flashMoeStatus(LauncherHandle(launcher), &bits, &launches, stream), 0);
  ASSERT_EQ(static_cast<int>(bits), 0);
  HIP_ERROR_ASSERT(hipFree(tokens_device));
  HIP_ERROR_ASSERT(hipFree(finalOutput_device));
  HIP_ERROR_ASSERT(DestroyLauncher(launcher, stream));
  printf("Moe kernel avg time for num of tokens: %d (%s) is %.4f ms.\n", numTokens,
         w.bf16 ? "bf16" : "float", avg_ms);
  fflush(stdout);
}

void FreeWeights(Weights& w) {
  hipFree(w.gate);
  hipFree(w.ffn1);
  hipFree(w.ffn2);
}

TEST(Benchmark, FlashMoeSingleGPU) {
  Weights w = MakeWeights(false);
  ASSERT_TRUE(w.gate && w.ffn1 && w.ffn2);
  for (int t : {1, 16, 32, 64, 256}) {
    PerformBenchmark(w, t, mini_ok);
    if (!mini_ok) return;
  }
  FreeWeights(w);
}

TEST(Benchmark, FlashMoeSingleGPUBf16) {
  Weights w = MakeWeights(true);
  ASSERT_TRUE(w.gate && w.ffn1 && w.ffn2);
  for (int t : {1, 64, 1024, 8192}) {
    PerformBenchmark(w, t, mini_ok);
    if (!mini_ok) return;
  }
  FreeWeights(w);
}

}  // namespace

int main() { return mini::run_all(); }
