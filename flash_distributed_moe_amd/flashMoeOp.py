"""A sparse-MoE block that runs on the fused launcher.

`FlashMoeBlockWrapper(block, maxTokens)` stands in for the Qwen3-MoE block it is
given, the way the reference's vLLM wrapper does
(test/singleGPU/python/flashMoeOp.py:7-38): same class name, same first two
constructor arguments, same attributes (`qwen3MoeSparseMoeBlockModule`,
`launcher`, `maxTokens`), result written over `hidden_states`. The launcher is
the compiled `flashMoeLauncher` extension; there is no fallback to Python code
when it has not been built.

What differs from the reference wrapper: float32 or bfloat16 weights of any
admitted shape (the reference: float32, the 30B shape only); `top_k` and a router
bias are taken from the block when it has them; a launch is one kernel, so
`forward` can be captured into a HIP graph; batches beyond `maxTokens` go to the
wrapped block itself (the reference calls `super().forward`, which
`torch.nn.Module` does not define). `pack_weights` says how the kernels get the
packed weight layout they read fastest: True (default) keeps a packed second
copy inside the launcher and leaves the block's tensors alone (that doubles the
memory of the block's expert weights: 1.1 GiB per layer of the 30B model, which
the library announces once per process; a 288 GB device holds the 30B model's 48
layers twice over, and the block stays usable as the fallback); "in_place"
rewrites the block's `w13_weight` / `w2_weight` into the packed layout where they
lie (no extra memory; the wrapped block can then no longer compute with them, so
`maxTokens` must cover every batch); False reads the row-major tensors.
"""
import os
import sys

import torch

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)
try:
    import flashMoeLauncher
except ImportError as e:  # no fallback: say how to build it
    raise ImportError("the flashMoeLauncher extension is not built; run "
                      "`python -m flash_distributed_moe_amd.build` (%s)" % e)


def _find_int(objs, names):
    for o in objs:
        for n in names:
            v = getattr(o, n, None)
            if isinstance(v, int) and v > 0:
                return v
    return None


class FlashMoeBlockWrapper(torch.nn.Module):

    def __init__(self, qwen3MoeSparseMoeBlockModule, maxTokens, top_k=None, router_bias=None,
                 pack_weights=True):
        super().__init__()
        block = qwen3MoeSparseMoeBlockModule
        self.qwen3MoeSparseMoeBlockModule = block
        self.maxTokens = int(maxTokens)
        if top_k is None:
            top_k = _find_int((block, getattr(block, "experts", None), getattr(block, "gate", None)),
                              ("top_k", "num_experts_per_tok")) or 8
        if router_bias is None:
            router_bias = getattr(block.gate, "bias", None)
        self.weights_in_place = pack_weights == "in_place"
        if self.weights_in_place:
            flashMoeLauncher.pack_weights_in_place(block.experts.w13_weight.data, block.experts.w2_weight.data)
            flags = flashMoeLauncher.FLAG_WEIGHTS_PREPACKED
        else:
            flags = flashMoeLauncher.FLAG_PACK_WEIGHTS if pack_weights else 0
        self.launcher = flashMoeLauncher.MoeKernelLauncher()
        self.launcher.create(
            block.gate.weight, block.experts.w13_weight, block.experts.w2_weight, self.maxTokens,
            self.launcher.getDistributedUniqueId(empty=True), 0, 1, top_k=int(top_k),
            router_bias=router_bias, flags=flags)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        if hidden_states.shape[0] > self.maxTokens:
            if self.weights_in_place:
                raise RuntimeError("batch of %d tokens exceeds maxTokens = %d and the wrapped block's "
                                   "weights were packed in place" % (hidden_states.shape[0], self.maxTokens))
            return self.qwen3MoeSparseMoeBlockModule(hidden_states)
        self.launcher.launch(hidden_states, hidden_states)  # output aliases input
        return hidden_states

    def __del__(self):
        launcher = getattr(self, "launcher", None)
        if launcher is not None and launcher.valid:
            launcher.destroy()
