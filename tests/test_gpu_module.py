"""The vLLM-shaped caller above the boundary: FlashMoeBlockWrapper on a stand-in
sparse-MoE block (vLLM is not installed), in place, with the large-batch
fallback, and captured into a HIP graph."""
import numpy as np
import pytest
import torch

from flash_distributed_moe_amd import synth
from flash_distributed_moe_amd.flashMoeOp import FlashMoeBlockWrapper
from oracle import oracle
from tests.helpers import max_rel_err

pytestmark = pytest.mark.gpu


class _Linear(torch.nn.Module):
    def __init__(self, weight):
        super().__init__()
        self.weight = torch.nn.Parameter(weight, requires_grad=False)


class _Experts(torch.nn.Module):
    def __init__(self, w13, w2, top_k):
        super().__init__()
        self.w13_weight = torch.nn.Parameter(w13, requires_grad=False)
        self.w2_weight = torch.nn.Parameter(w2, requires_grad=False)
        self.top_k = top_k


class StandInSparseMoeBlock(torch.nn.Module):
    """The attributes the wrapper reads from vLLM's Qwen3MoeSparseMoeBlock, and a
    forward of its own (plain torch) that marks its output so a test can tell
    which path ran."""

    def __init__(self, inp, top_k):
        super().__init__()
        self.gate = _Linear(inp["gate"])
        self.experts = _Experts(inp["ffn1"], inp["ffn2"], top_k)
        self.calls = 0

    def forward(self, hidden_states):
        self.calls += 1
        return torch.full_like(hidden_states, 7.0)


def _oracle_out(cfg, inp, x):
    f = lambda t: t.float().cpu().numpy()
    return oracle.forward(f(x), f(inp["gate"]), f(inp["ffn1"]), f(inp["ffn2"]), cfg.k)[0]


@pytest.mark.parametrize("name,T", [("tiny_f32", 16), ("qwen3_30b_decode", 24)])
def test_wrapper_in_place_and_fallback(name, T):
    cfg = synth.CONFIGS[name].replace(T=T)
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, 7907, dev)
    block = StandInSparseMoeBlock(inp, cfg.k)
    layer = FlashMoeBlockWrapper(block, maxTokens=T)
    x = inp["tokens"].clone()
    ref = _oracle_out(cfg, inp, x)
    y = layer(x)
    torch.cuda.synchronize()
    assert y.data_ptr() == x.data_ptr(), "forward must work in place"
    tol = 1e-2 if cfg.dtype == "bf16" else 2e-5
    assert max_rel_err(y.float().cpu().numpy(), ref) <= tol
    assert block.calls == 0
    # more tokens than maxTokens: the wrapped block runs instead
    big = torch.cat([inp["tokens"], inp["tokens"]], 0)
    z = layer(big)
    torch.cuda.synchronize()
    assert block.calls == 1 and float(z[0, 0]) == 7.0
    del layer


@pytest.mark.parametrize("T", [32, 512])
def test_forward_in_hip_graph(T):
    """A launch is one kernel and touches no host state, so it can be captured.
    Every replay gets fresh token contents and is checked bit for bit against an
    eager launch of another launcher on the same input, with eager work and
    synchronisation between replays. 32 tokens run the streaming variant, 512 the
    tiled one (whose scratch rows are read with plain cached loads: a stale line
    from the previous replay would show here)."""
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=T)
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, 7907, dev)
    block = StandInSparseMoeBlock(inp, cfg.k)
    layer = FlashMoeBlockWrapper(block, maxTokens=cfg.T)
    eager = FlashMoeBlockWrapper(block, maxTokens=cfg.T)
    static_x = inp["tokens"].clone()
    # warm-up on a side stream, as torch's capture rules ask
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        layer(static_x.clone())
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    work = static_x.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        work.copy_(static_x)
        layer(work)
    for rep in range(4):
        fresh = synth.make_inputs_torch(cfg, 100 + rep, dev)["tokens"]
        static_x.copy_(fresh)
        g.replay()
        torch.cuda.synchronize()
        want = eager(fresh.clone())
        torch.cuda.synchronize()
        assert torch.equal(work, want), "replay %d differs from the eager launch" % rep
        if rep == 0:
            ref = _oracle_out(cfg, inp, fresh)
            assert max_rel_err(work.float().cpu().numpy(), ref) <= 1e-2
    del layer, eager


def test_python_binding_sequence_of_the_reference():
    """The create / launch / destroy sequence of the reference's
    test/singleGPU/python/test_pythonBinding.py:5-40, under the same import,
    float32 at the reference's shape, plus what that test leaves out: the
    result is checked against the oracle."""
    import flashMoeLauncher

    cfg = synth.MoeConfig("binding", 16, 2048, 128, 8, 768, "f32")
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, 123, dev)
    tokens = inp["tokens"]
    output = torch.empty_like(tokens)
    launcher = flashMoeLauncher.MoeKernelLauncher()
    assert launcher.valid == False  # noqa: E712
    uniqueid = launcher.getDistributedUniqueId(empty=True)
    launcher.create(inp["gate"], inp["ffn1"], inp["ffn2"], cfg.T, uniqueid, 0, 1)
    assert launcher.valid == True  # noqa: E712
    launcher.launch(tokens, output)
    torch.cuda.synchronize(dev)
    assert output.shape == (cfg.T, cfg.H) and output.dtype == torch.float32
    assert max_rel_err(output.cpu().numpy(), _oracle_out(cfg, inp, tokens)) <= 2e-5
    with pytest.raises(RuntimeError, match="output shape"):
        launcher.launch(tokens, output[:4])
    launcher.destroy()
    assert launcher.valid == False  # noqa: E712
    with pytest.raises(RuntimeError, match="Launcher was destroyed"):
        launcher.launch(tokens, output)
    # beyond the reference's surface: the pre-norm block's MoE half in one call
    gamma = torch.linspace(0.5, 1.5, cfg.H, device=dev)
    launcher.create(inp["gate"], inp["ffn1"], inp["ffn2"], cfg.T, uniqueid, 0, 1,
                    flags=flashMoeLauncher.FLAG_RMSNORM | flashMoeLauncher.FLAG_RESIDUAL,
                    norm_weight=gamma, norm_eps=1e-6)
    launcher.launch(tokens, output)
    torch.cuda.synchronize(dev)
    f = lambda t: t.float().cpu().numpy()
    want = oracle.layer(f(tokens), f(inp["gate"]), f(inp["ffn1"]), f(inp["ffn2"]), cfg.k,
                        norm_weight=f(gamma), norm_eps=1e-6, residual=True)[0]
    assert max_rel_err(output.cpu().numpy(), want) <= 2e-5
    with pytest.raises(RuntimeError, match="norm_weight"):
        flashMoeLauncher.MoeKernelLauncher().create(inp["gate"], inp["ffn1"], inp["ffn2"], cfg.T, uniqueid, 0, 1,
                                                    flags=flashMoeLauncher.FLAG_RMSNORM)
    launcher.destroy()


def test_wrapper_packs_the_blocks_weights_in_place():
    """pack_weights="in_place": the block's expert tensors are rewritten into the
    packed layout (no second copy); results as with the row-major tensors, and a
    batch beyond maxTokens is an error instead of a wrong answer from the wrapped block."""
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=24)
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, 7907, dev)
    mine = dict(inp, ffn1=inp["ffn1"].clone(), ffn2=inp["ffn2"].clone())
    layer = FlashMoeBlockWrapper(StandInSparseMoeBlock(mine, cfg.k), maxTokens=cfg.T, pack_weights="in_place")
    assert not torch.equal(mine["ffn1"], inp["ffn1"])
    plain = FlashMoeBlockWrapper(StandInSparseMoeBlock(inp, cfg.k), maxTokens=cfg.T, pack_weights=False)
    x = inp["tokens"]
    got, want = layer(x.clone()), plain(x.clone())
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert max_rel_err(got.float().cpu().numpy(), _oracle_out(cfg, inp, x)) <= 1e-2
    with pytest.raises(RuntimeError, match="packed in place"):
        layer(torch.cat([x, x], 0))
    del layer, plain


@pytest.mark.parametrize("name,T", [("qwen3_30b_decode", 64), ("qwen3_30b_decode", 700), ("tiny_f32", 16)])
def test_extension_and_ctypes_mirror_agree(name, T):
    """The compiled `flashMoeLauncher` extension (what callers import) and the ctypes class the
    parity tests drive end in the same C entry points: same bits for the same call, with the
    defaults of both (`create` without flags: the launcher's packed copy), and the same refusals."""
    import flashMoeLauncher as ext
    from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher as Mirror

    cfg = synth.CONFIGS[name].replace(T=T)
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, 31, dev)
    x = inp["tokens"]
    outs = []
    for cls in (ext.MoeKernelLauncher, Mirror):
        l = cls()
        uid = l.getDistributedUniqueId(empty=True)
        assert bytes(uid) == bytes(128)
        l.create(inp["gate"], inp["ffn1"], inp["ffn2"], cfg.T, uid, 0, 1, top_k=cfg.k)
        out = torch.full_like(x, float("nan"))
        l.launch(x, out)
        torch.cuda.synchronize()
        outs.append(out.clone())
        for bad in (lambda: l.launch(x, out[:1]),                      # shapes differ
                    lambda: l.launch(x.float() if x.dtype != torch.float32 else x.bfloat16(), out)):  # dtype
            with pytest.raises((RuntimeError, ValueError, TypeError)):
                bad()
        l.destroy()
        assert not l.valid
        with pytest.raises(RuntimeError, match="Launcher was destroyed"):
            l.launch(x, out)
        with pytest.raises((RuntimeError, ValueError)):
            cls().create(inp["gate"], inp["ffn1"], inp["ffn2"], cfg.T, uid, 1, 2, top_k=cfg.k)  # world size 2
    assert torch.equal(outs[0], outs[1])
