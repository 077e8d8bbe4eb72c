"""The two optional steps at the layer's edges, through the C ABI against the oracle:
FLASH_MOE_FLAG_RMSNORM (the layer runs on rmsnorm(tokens)) and FLASH_MOE_FLAG_RESIDUAL
(the input rows are added to the output), alone and together, out of place and in place,
on the streaming and on the tiled variant. Routing after the norm must stay bit-exact:
the normalised rows are defined to the last rounding. Outputs to moe_case.TOL."""
import numpy as np
import pytest
import torch

from flash_distributed_moe_amd import _lib, synth
from tests.moe_case import GpuCase

pytestmark = pytest.mark.gpu

CASES = [("tiny_f32", 16, _lib.SCHED_STREAM), ("qwen3_30b_decode", 24, _lib.SCHED_STREAM),
         ("qwen3_30b_decode", 130, _lib.SCHED_TILED), ("qwen3_30b_decode", 700, _lib.SCHED_TILED)]


def _gamma(cfg, dev):
    dt = torch.bfloat16 if cfg.dtype == "bf16" else torch.float32
    return synth.normal_torch(5, 9, (cfg.H,), 0.25, torch.float32, dev).add_(1.0).to(dt)


def _rows(cfg, dev):
    """Token rows as a residual stream carries them: row scales spread over two decades."""
    x = synth.make_inputs_torch(cfg, 31, dev)["tokens"].float()
    scale = torch.logspace(-1, 1, cfg.T, device=dev).unsqueeze(1)
    return (x * scale).to(torch.bfloat16 if cfg.dtype == "bf16" else torch.float32)


@pytest.mark.parametrize("norm,residual", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("name,T,sched", CASES)
def test_norm_and_residual(name, T, sched, norm, residual):
    cfg = synth.CONFIGS[name].replace(T=T)
    print("case", name, "T", T, "sched", sched, "norm", norm, "residual", residual, flush=True)
    dev = torch.device("cuda:0")
    case = GpuCase(cfg, 31, sched, norm_weight=_gamma(cfg, dev) if norm else None, norm_eps=1e-5,
                   residual=residual)
    try:
        x = _rows(cfg, dev) if norm else case.inp["tokens"]
        out = case.run(x)
        case.check_routing(x, case.launcher.routing(T))
        case.check_outputs(x, out)
        again = case.run(x, inplace=True)
        assert torch.equal(again, out), "in place differs from out of place"
        # a smaller batch next, through the same workspace
        if T > 8:
            part = case.run(x[: T // 3].contiguous())
            case.check_outputs(x[: T // 3], part)
    finally:
        case.close()


def test_norm_needs_its_weight():
    cfg = synth.CONFIGS["tiny_f32"]
    d = _lib.LayerDesc()
    d.experts, d.hidden, d.intermediate, d.top_k = cfg.E, cfg.H, cfg.I, cfg.k
    d.dtype, d.max_tokens, d.flags = _lib.F32, 16, _lib.FLAG_RMSNORM
    import ctypes

    inp = synth.make_inputs_torch(cfg, 1, torch.device("cuda:0"))
    d.gate_weights, d.ffn1_weights, d.ffn2_weights = (inp[k].data_ptr() for k in ("gate", "ffn1", "ffn2"))
    h = ctypes.c_void_p()
    assert _lib.load().flashMoeCreate(ctypes.byref(h), ctypes.byref(d), None) == _lib.HIP_ERROR_INVALID_VALUE
