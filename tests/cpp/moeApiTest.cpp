// The reference's API test (test/singleGPU/cpp/moe/moeApiTest.cpp:5-12)
// re-targeted at this library: a batch beyond the launcher's capacity is refused
// with hipErrorUnknown before any pointer is looked at. The capacity is
// max_tokens * top_k <= 2^21 here (the reference: about 85 tokens), so the
// request is sized past that. Needs no GPU.
#include "include/iMoeKernelLauncher.h"
#include "tests/cpp/mini_test.h"

namespace {

TEST(MoeApiTests, maxHandledTokens) {
  const int TOKENS_NUM = (1 << 21) / 8 + 1;
  const moe::DistributedUniqueId duid = GetDistributedUniqueId(/*empty=*/true);
  moe::IMoeKernelLauncher* launcher = nullptr;
  ASSERT_EQ(CreateLauncher(&launcher, nullptr, nullptr, nullptr, TOKENS_NUM, nullptr, duid, 0, 1),
            hipErrorUnknown);
  ASSERT_TRUE(launcher == nullptr);
}

TEST(MoeApiTests, uniqueIdIsZeros) {
  for (bool empty : {true, false}) {
    const moe::DistributedUniqueId duid = GetDistributedUniqueId(empty);
    for (unsigned char b : duid.data) ASSERT_EQ(static_cast<int>(b), 0);
  }
}

TEST(MoeApiTests, oneGpuOnly) {
  const moe::DistributedUniqueId duid = GetDistributedUniqueId(/*empty=*/true);
  moe::IMoeKernelLauncher* launcher = nullptr;
  ASSERT_EQ(CreateLauncher(&launcher, nullptr, nullptr, nullptr, 16, nullptr, duid, 0, 2),
            hipErrorInvalidValue);
  ASSERT_EQ(CreateLauncher(&launcher, nullptr, nullptr, nullptr, 16, nullptr, duid, 1, 1),
            hipErrorInvalidValue);
  ASSERT_TRUE(launcher == nullptr);
}

}  // namespace

int main() { return mini::run_all(); }
