"""The entry point that allocates nothing (flashMoeLaunchNoAlloc) against
flashMoeCreate + flashMoeLaunch on the same inputs: same kernels, so the outputs
must be equal bit for bit; two calls in a row on the shared static workspace,
the second with a smaller batch and another shape, then the first again."""
import ctypes

import numpy as np
import pytest
import torch

from flash_distributed_moe_amd import _lib, synth
from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher
from oracle import oracle
from tests.helpers import max_rel_err

pytestmark = pytest.mark.gpu


def layer_desc(cfg, inp, max_tokens, sched):
    d = _lib.LayerDesc()
    d.experts, d.hidden, d.intermediate, d.top_k = cfg.E, cfg.H, cfg.I, cfg.k
    d.dtype = _lib.BF16 if cfg.dtype == "bf16" else _lib.F32
    d.max_tokens, d.sched, d.flags = max_tokens, sched, 0
    d.gate_weights = inp["gate"].data_ptr()
    d.ffn1_weights = inp["ffn1"].data_ptr()
    d.ffn2_weights = inp["ffn2"].data_ptr()
    d.router_bias = inp["bias"].data_ptr() if inp["bias"] is not None else None
    return d


def no_alloc(cfg, inp, x, sched, inplace=False):
    lib = _lib.load()
    d = layer_desc(cfg, inp, x.shape[0], sched)
    out = x.clone() if inplace else torch.full_like(x, float("nan"))
    src = out if inplace else x
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.flashMoeLaunchNoAlloc(ctypes.byref(d), src.data_ptr(), out.data_ptr(), x.shape[0], stream)
    assert rc == _lib.HIP_SUCCESS, "flashMoeLaunchNoAlloc returned %d" % rc
    torch.cuda.synchronize()
    return out


def with_launcher(cfg, inp, x, sched):
    l = MoeKernelLauncher()
    l.create(inp["gate"], inp["ffn1"], inp["ffn2"], x.shape[0], l.getDistributedUniqueId(True), 0, 1,
             top_k=cfg.k, router_bias=inp["bias"], sched=sched)
    try:
        out = torch.full_like(x, float("nan"))
        l.launch(x, out)
        torch.cuda.synchronize()
        assert l.status()[0] == 0
        return out
    finally:
        l.destroy()


def launcher_sched(cfg, inp, T, sched):
    """AUTO falls back to the streaming variant when the workspace of the variant
    flashMoeLaunch would take does not fit the static array."""
    n = ctypes.c_size_t(0)
    d = layer_desc(cfg, inp, T, sched)
    assert _lib.load().flashMoeWorkspaceBytes(ctypes.byref(d), ctypes.byref(n)) == 0
    return _lib.SCHED_STREAM if n.value > _lib.NOALLOC_SCRATCH_BYTES else sched


def oracle_out(cfg, inp, x):
    f = lambda t: None if t is None else t.float().cpu().numpy()
    ref, _, _ = oracle.forward(f(x), f(inp["gate"]), f(inp["ffn1"]), f(inp["ffn2"]), cfg.k, bias=f(inp["bias"]))
    return ref


def test_no_alloc_equals_launcher_two_calls_in_a_row():
    dev = torch.device("cuda:0")
    big = synth.CONFIGS["qwen3_30b_decode"].replace(T=48, name="decode48")
    small = synth.CONFIGS["tiny_f32"]
    inp_big = synth.make_inputs_torch(big, 7907, dev)
    inp_small = synth.make_inputs_torch(small, 11, dev)
    for sched in (_lib.SCHED_STREAM, _lib.SCHED_AUTO):
        print("no-alloc, sched", sched, flush=True)
        # first call: 48 tokens of the 30B shape; second: a smaller batch of the same layer;
        # third: another (tiny, float32) layer; fourth: the first again on whatever those left
        xs = [(big, inp_big, inp_big["tokens"]), (big, inp_big, inp_big["tokens"][:5].contiguous()),
              (small, inp_small, inp_small["tokens"]), (big, inp_big, inp_big["tokens"])]
        got = [no_alloc(c, i, x, sched) for c, i, x in xs]
        for (c, i, x), g in zip(xs, got):
            want = with_launcher(c, i, x, launcher_sched(c, i, x.shape[0], sched))
            assert torch.equal(g, want), "%s T=%d differs from flashMoeLaunch" % (c.name, x.shape[0])
            tol = 1e-2 if c.dtype == "bf16" else 2e-5
            err = max_rel_err(g.float().cpu().numpy(), oracle_out(c, i, x))
            print("  %s T=%d: equal to the launcher's output, max rel err vs oracle %.2e" % (c.name, x.shape[0], err),
                  flush=True)
            assert err <= tol
        assert torch.equal(got[0], got[3])
    # in place, as the reference's callers run it
    g = no_alloc(big, inp_big, inp_big["tokens"], _lib.SCHED_STREAM, inplace=True)
    assert torch.equal(g, no_alloc(big, inp_big, inp_big["tokens"], _lib.SCHED_STREAM))


def test_no_alloc_with_norm_and_residual():
    """The optional RMSNorm / residual steps use the static workspace too (the normalised
    rows live there): same bits as the launcher with the same flags."""
    dev = torch.device("cuda:0")
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=40, name="decode40")
    inp = synth.make_inputs_torch(cfg, 7907, dev)
    gamma = synth.normal_torch(5, 9, (cfg.H,), 0.25, torch.float32, dev).add_(1.0).to(torch.bfloat16)
    lib = _lib.load()
    for T in (40, 7):
        x = inp["tokens"][:T].contiguous()
        d = layer_desc(cfg, inp, T, _lib.SCHED_AUTO)
        d.flags = _lib.FLAG_RMSNORM | _lib.FLAG_RESIDUAL
        d.norm_weight, d.norm_eps = gamma.data_ptr(), 1e-6
        out = torch.full_like(x, float("nan"))
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.flashMoeLaunchNoAlloc(ctypes.byref(d), x.data_ptr(), out.data_ptr(), T, stream) == 0
        torch.cuda.synchronize()
        l = MoeKernelLauncher()
        l.create(inp["gate"], inp["ffn1"], inp["ffn2"], T, l.getDistributedUniqueId(True), 0, 1, top_k=cfg.k,
                 router_bias=inp["bias"], norm_weight=gamma, norm_eps=1e-6, residual=True)
        try:
            want = torch.full_like(x, float("nan"))
            l.launch(x, want)
            torch.cuda.synchronize()
        finally:
            l.destroy()
        assert torch.equal(out, want)
        f = lambda t: None if t is None else t.float().cpu().numpy()
        ref = oracle.layer(f(x), f(inp["gate"]), f(inp["ffn1"]), f(inp["ffn2"]), cfg.k, bias=f(inp["bias"]),
                           norm_weight=f(gamma), norm_eps=1e-6, residual=True, bf16=True)[0]
        assert max_rel_err(out.float().cpu().numpy(), ref) <= 1e-2


def test_no_alloc_rejects_what_does_not_fit(capfd):
    dev = torch.device("cuda:0")
    cfg = synth.CONFIGS["qwen3_30b_decode"]
    inp = synth.make_inputs_torch(cfg, 7907, dev)
    lib = _lib.load()
    T = 4096
    x = torch.zeros(T, cfg.H, dtype=torch.bfloat16, device=dev)
    out = torch.full_like(x, 1.0)
    d = layer_desc(cfg, inp, T, _lib.SCHED_AUTO)
    rc = lib.flashMoeLaunchNoAlloc(ctypes.byref(d), x.data_ptr(), out.data_ptr(), T, None)
    torch.cuda.synchronize()
    assert rc == _lib.HIP_ERROR_UNKNOWN
    assert "static one holds" in capfd.readouterr().out
    assert bool((out == 1.0).all())            # nothing ran
    d = layer_desc(cfg, inp, 8, _lib.SCHED_AUTO)
    assert lib.flashMoeLaunchNoAlloc(ctypes.byref(d), x.data_ptr(), out.data_ptr(), 9, None) == _lib.HIP_ERROR_UNKNOWN
    d.flags = _lib.FLAG_PACK_WEIGHTS
    assert lib.flashMoeLaunchNoAlloc(ctypes.byref(d), x.data_ptr(), out.data_ptr(), 8, None) == _lib.HIP_ERROR_INVALID_VALUE


def test_no_alloc_status_and_graph_capture():
    """After a warm-up call (which looks up the static array's address) the call can be
    recorded into a HIP graph: it allocates nothing and enqueues kernels only. Every replay
    gets fresh tokens and must equal an eager launcher's result; flashMoeNoAllocStatus
    reports no device error after them."""
    lib = _lib.load()
    dev = torch.device("cuda:0")
    for T, sched in ((40, _lib.SCHED_STREAM), (600, _lib.SCHED_TILED)):
        cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=T, name="graph%d" % T)
        inp = synth.make_inputs_torch(cfg, 7907, dev)
        d = layer_desc(cfg, inp, T, sched)
        static_x = inp["tokens"].clone()
        static_out = torch.empty_like(static_x)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # warm-up outside the capture
            rc = lib.flashMoeLaunchNoAlloc(ctypes.byref(d), static_x.data_ptr(), static_out.data_ptr(), T,
                                           ctypes.c_void_p(side.cuda_stream))
            assert rc == _lib.HIP_SUCCESS
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            rc = lib.flashMoeLaunchNoAlloc(ctypes.byref(d), static_x.data_ptr(), static_out.data_ptr(), T,
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            assert rc == _lib.HIP_SUCCESS
        for rep in range(3):
            fresh = synth.normal_torch(500 + rep, synth.STREAM_TOKENS, (T, cfg.H), 1.0, torch.bfloat16, dev)
            static_x.copy_(fresh)
            g.replay()
            torch.cuda.synchronize()
            want = with_launcher(cfg, inp, fresh, sched)   # eager work between the replays
            assert torch.equal(static_out, want), "replay %d of the recorded no-alloc call differs" % rep
        bits = ctypes.c_uint(99)
        assert lib.flashMoeNoAllocStatus(ctypes.byref(bits), None) == _lib.HIP_SUCCESS
        assert bits.value == 0
        print("  no-alloc call recorded and replayed three times, T=%d sched=%d" % (T, sched), flush=True)
