// C++ launcher interface of the fused MoE layer, binary compatible with the
// reference's include/iMoeKernelLauncher.h:9-39 (same abstract class and
// vtable order, same three extern "C" symbols with the same parameter lists),
// so callers written against the reference link against this library
// unchanged. The shape-carrying CreateLauncherEx is an addition: the reference
// fixes E=128, H=2048, I=768, top-8, float at compile time
// (src/hip/common/metadata.h:7-13) and CreateLauncher keeps meaning exactly that.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flash_moe.h"

namespace moe {

class IMoeKernelLauncher {
 public:
  // Enqueues one forward pass over tokens[tokensNum, H] on `stream`; does not
  // wait. `output` may be the same buffer as `tokens`.
  virtual hipError_t Launch(const void* tokens, void* output, int tokensNum,
                            hipStream_t stream) = 0;
  virtual ~IMoeKernelLauncher();
};

// Kept for signature compatibility; this library has no inter-GPU transport,
// so the id is always 128 zero bytes.
struct DistributedUniqueId {
  uint8_t data[128];
};

}  // namespace moe

extern "C" moe::DistributedUniqueId GetDistributedUniqueId(bool empty);

// Reference shape (E128, H2048, I768, top-8, float). Only rank 0 of a world of
// 1 is supported; anything else returns hipErrorInvalidValue.
extern "C" hipError_t CreateLauncher(moe::IMoeKernelLauncher** launcher, const void* gateWeights,
                                     const void* ffn1ExpertWeights,
                                     const void* ffn2ExpertWeights, int maxTokens,
                                     hipStream_t stream, const moe::DistributedUniqueId& uid,
                                     int rank, int worldSize);

// Any supported shape / dtype / top-k, optional router bias.
extern "C" hipError_t CreateLauncherEx(moe::IMoeKernelLauncher** launcher,
                                       const FlashMoeLayerDesc* desc, hipStream_t stream);

extern "C" hipError_t DestroyLauncher(moe::IMoeKernelLauncher* launcher, hipStream_t stream);

// The C handle behind a launcher made by CreateLauncher / CreateLauncherEx (for
// flashMoeReadRouting and flashMoeStatus).
extern "C" FlashMoeLauncher* LauncherHandle(moe::IMoeKernelLauncher* launcher);
