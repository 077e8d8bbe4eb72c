"""torch.nn.Module over the fused MoE launcher, shaped like the reference's
vLLM wrapper (test/singleGPU/python/flashMoeOp.py:7-38): it takes the sparse
MoE block of a Qwen3-MoE model, borrows `gate.weight`, `experts.w13_weight`
and `experts.w2_weight`, runs the layer in place on `hidden_states`, and hands
batches larger than `maxTokens` to the wrapped block.

Differences from the reference wrapper: float32 and bfloat16 weights of any
admitted shape (the reference: float32, the 30B shape only); `top_k` and an
optional router bias are read from the block when it has them; a launch is a
single kernel, so `forward` can be captured into a HIP graph; the fallback calls
the wrapped block (the reference calls `super().forward`, which
`torch.nn.Module` does not implement).
"""
import torch

from . import flashMoeLauncher


def _block_top_k(block, default=8):
    for owner in (block, getattr(block, "experts", None), getattr(block, "gate", None)):
        for name in ("top_k", "num_experts_per_tok"):
            v = getattr(owner, name, None)
            if isinstance(v, int) and v > 0:
                return v
    return default


class FlashMoeBlockWrapper(torch.nn.Module):

    def __init__(self, qwen3MoeSparseMoeBlockModule, maxTokens, top_k=None, router_bias=None,
                 pack_weights=False):
        super().__init__()
        self.qwen3MoeSparseMoeBlockModule = qwen3MoeSparseMoeBlockModule
        self.launcher = flashMoeLauncher.MoeKernelLauncher()

        gateWeights = self.qwen3MoeSparseMoeBlockModule.gate.weight
        ffn1ExpertWeights = self.qwen3MoeSparseMoeBlockModule.experts.w13_weight
        ffn2ExpertWeights = self.qwen3MoeSparseMoeBlockModule.experts.w2_weight
        if router_bias is None:
            router_bias = getattr(self.qwen3MoeSparseMoeBlockModule.gate, "bias", None)

        uniqueid = self.launcher.getDistributedUniqueId(empty=True)
        self.launcher.create(
            gateWeights, ffn1ExpertWeights, ffn2ExpertWeights, maxTokens, uniqueid, 0, 1,
            top_k=top_k if top_k is not None else _block_top_k(qwen3MoeSparseMoeBlockModule),
            router_bias=router_bias, pack_weights=pack_weights,
        )
        self.maxTokens = maxTokens

    def __del__(self):
        launcher = getattr(self, "launcher", None)
        if launcher is not None and launcher.valid:
            launcher.destroy()

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        num_tokens, _ = hidden_states.shape

        if num_tokens <= self.maxTokens:
            tokens = hidden_states

            # Inplace calc -> output_mem = input_mem
            self.launcher.launch(tokens, tokens)

            return tokens
        else:
            return self.qwen3MoeSparseMoeBlockModule(hidden_states)
