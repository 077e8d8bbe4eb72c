"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on
the same seeded inputs. Routing (top-k indices, expert counts/offsets,
permutation) must be bit-exact; outputs within the tolerance in moe_case.TOL."""
import numpy as np
import pytest
import torch

from flash_distributed_moe_amd import _lib, synth
from tests.moe_case import GpuCase

pytestmark = pytest.mark.gpu


def run_case(cfg, seed=7907, sched=_lib.SCHED_STREAM, sample=None, inplace=False):
    print("case", cfg.name, "T", cfg.T, "H", cfg.H, "E", cfg.E, "k", cfg.k, "I", cfg.I,
          cfg.dtype, "seed", seed, "sched", sched, flush=True)
    case = GpuCase(cfg, seed, sched)
    try:
        x = case.inp["tokens"]
        out = case.run(inplace=inplace)
        routing = case.launcher.routing(cfg.T)
        case.check_routing(x, routing)
        ids = None
        if sample is not None and sample < cfg.T:
            ids = np.unique(np.linspace(0, cfg.T - 1, sample).astype(np.int64))
        err = case.check_outputs(x, out, ids)
        print("  max rel err %.3e" % err, flush=True)
        return case, out
    finally:
        case.close()


def test_tiny_f32():
    run_case(synth.CONFIGS["tiny_f32"])


def test_tiny_f32_matches_golden(golden_dir):
    import os

    g = np.load(os.path.join(golden_dir, "ref_tiny_f32.npz"))
    cfg = synth.CONFIGS["tiny_f32"]
    case = GpuCase(cfg, int(g["seed"]))
    try:
        out = case.run().cpu().numpy()
        r = case.launcher.routing(cfg.T)
        assert np.array_equal(r["topk_idx"], g["topk_idx"])
        np.testing.assert_allclose(r["topk_w"], g["topk_w"], rtol=2e-6)
        assert np.max(np.abs(out - g["out"])) <= 2e-5 * np.max(np.abs(g["out"]))
    finally:
        case.close()


# AUTO takes the streaming variant at this size; the tiled one is asked for by name
@pytest.mark.parametrize("seed,sched", [(7907, _lib.SCHED_STREAM), (1, _lib.SCHED_STREAM),
                                        (2, _lib.SCHED_STREAM), (7907, _lib.SCHED_AUTO), (7907, _lib.SCHED_TILED)])
def test_qwen3_30b_decode(seed, sched):
    run_case(synth.CONFIGS["qwen3_30b_decode"], seed=seed, sched=sched)


@pytest.mark.parametrize("sched", [_lib.SCHED_STREAM, _lib.SCHED_TILED])
def test_qwen3_30b_decode_inplace(sched):
    run_case(synth.CONFIGS["qwen3_30b_decode"], inplace=True, sched=sched)


@pytest.mark.parametrize("sched", [_lib.SCHED_STREAM, _lib.SCHED_TILED])
@pytest.mark.parametrize("T", [1, 3, 17, 65, 130])
def test_ragged_token_counts_bf16(T, sched):
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=T, name="ragged")
    run_case(cfg, seed=T, sched=sched)


@pytest.mark.parametrize("shape", [
    # T, H, E, k, I, dtype
    (5, 64, 16, 4, 32, "f32"),
    (7, 128, 8, 8, 64, "f32"),      # k == E
    (33, 256, 32, 1, 96, "bf16"),   # top-1
    (40, 192, 200, 6, 160, "bf16"),  # E not a multiple of 64
    (100, 64, 4, 2, 32, "bf16"),    # > 64 rows per expert: several row tiles
    (64, 64, 4, 2, 32, "bf16"),     # small batch whose experts get ~32 rows: early tasks re-run with more row blocks
    (48, 128, 2, 1, 64, "bf16"),    # ~24 rows per expert, top-1
    (60, 128, 3, 3, 64, "f32"),     # k == E: 60 rows in every expert
])
def test_odd_shapes(shape):
    T, H, E, k, I, dt = shape
    run_case(synth.MoeConfig("odd", T, H, E, k, I, dt), seed=T + H)


@pytest.mark.parametrize("shape", [
    # T, H, E, k, I, hot: bf16 layers with H % 256 == 0 run the logit chains on the
    # matrix core, 16 tokens x 16 experts per workgroup, in stages of 256 k whose
    # loads go out eight stages at a time
    (17, 768, 24, 3, 64, 0),      # three stages; last token group and last expert group partly empty
    (65, 2304, 60, 5, 96, 0),     # nine stages: a second, short batch of loads
    (130, 512, 200, 6, 160, 0),   # 9 x 13 groups
    (1, 4096, 16, 2, 64, 0),      # one token, sixteen stages
    (200, 1024, 48, 4, 64, 3),    # router bias
    (40, 768, 24, 3, 64, 0),      # early gate/up tasks (T <= 64, T*k >= E) behind the same router
    (64, 512, 72, 8, 32, 2),      # the same with 4.5 expert groups and a bias
    (60, 256, 16, 2, 64, 2),      # early tasks; the two hot experts hold far more than 16 rows and start over
    (150, 512, 128, 8, 64, 0),    # early tasks behind three 64-token mask words
    (150, 256, 64, 4, 64, 1),     # early tasks; the hot expert holds all 150 tokens: its one tile is walked in 64-row steps
    (100, 512, 128, 8, 32, 2),    # the same with two hot experts of 100 rows
    (250, 512, 128, 8, 64, 0),    # 12 to 24 rows per expert: early tasks of two row blocks
    (230, 256, 64, 4, 64, 1),     # the same with a hot expert of 230 rows
])
def test_matrix_core_router_shapes(shape):
    T, H, E, k, I, hot = shape
    run_case(synth.MoeConfig("mcr", T, H, E, k, I, "bf16", hot=hot), seed=T + E)


def test_router_bias_hot_experts_small():
    cfg = synth.MoeConfig("hot", 256, 256, 16, 4, 64, "bf16", hot=2)
    run_case(cfg, seed=3)


def test_relaunch_and_smaller_batch():
    """Counters return to zero by themselves: launch twice, then a smaller batch."""
    cfg = synth.CONFIGS["qwen3_30b_decode"]
    case = GpuCase(cfg, sched=_lib.SCHED_STREAM)
    try:
        x = case.inp["tokens"]
        a = case.run()
        b = case.run()
        assert torch.equal(a, b)
        small = x[:20].contiguous()
        c = case.run(tokens=small)
        r = case.launcher.routing(20)
        case.check_routing(small, r)
        assert torch.equal(c, a[:20])       # tokens are independent
        assert case.launcher.status() == (0, 3)
    finally:
        case.close()


@pytest.mark.parametrize("sched", [_lib.SCHED_STREAM, _lib.SCHED_AUTO])
def test_relaunch_across_batch_sizes(sched):
    """One launcher, batches that take different paths one after the other (early
    gate/up tasks, the ordinary ticket order, one token, and with AUTO the tiled
    variant): every launch leaves the counters as the next one needs them."""
    cfg = synth.MoeConfig("seq", 600, 512, 64, 4, 128, "bf16")
    case = GpuCase(cfg, seed=11, sched=sched)
    try:
        x = case.inp["tokens"]
        full = case.run()
        case.check_routing(x, case.launcher.routing(cfg.T))
        case.check_outputs(x, full, np.arange(0, cfg.T, 7))
        for T in (150, 600, 40, 1, 190, 300, 64):
            part = x[:T].contiguous()
            out = case.run(tokens=part)
            case.check_routing(part, case.launcher.routing(T))
            case.check_outputs(part, out, np.arange(0, T, 3))
        assert case.launcher.status()[0] == 0
    finally:
        case.close()


@pytest.mark.parametrize("shape", [
    # T, H, E, k, I: the tiled (MFMA 32x32, LDS-staged) variant forced on small problems
    (300, 256, 8, 2, 128),      # ragged last row tile (75 rows per expert on average)
    (700, 512, 4, 2, 256),      # several 256-row tiles per expert, ragged tail
    (64, 256, 200, 6, 128),     # E > 128: two expert slabs in the router; tiny tiles
    (1, 256, 8, 2, 128),        # a single token
    (1100, 256, 8, 2, 128),     # ~275 rows per expert: tall tiles (a tail of <= 64 rows joins the full tile)
    (1180, 512, 4, 1, 256),     # ~295 rows per expert, top-1; some experts beyond 320 rows (tile + tail tile)
    (4100, 256, 200, 6, 128),   # more than one round of 16-token router tasks: 32-token tasks, two expert slabs, ragged last task
    (900, 768, 8, 2, 384),      # twelve and six 64-k stages: the packed weights' deeper pipeline past its first and last stages
    (2500, 512, 8, 1, 640),     # ~312 rows per expert: tiles of nine and ten 32-row blocks on three token buffers
])
def test_tiled_variant_forced(shape):
    T, H, E, k, I = shape
    cfg = synth.MoeConfig("tiled", T, H, E, k, I, "bf16")
    print("tiled forced", shape, flush=True)
    case = GpuCase(cfg, seed=T + E, sched=_lib.SCHED_TILED)
    try:
        assert case.launcher.sched_for(T) == _lib.SCHED_TILED
        x = case.inp["tokens"]
        out = case.run()
        case.check_routing(x, case.launcher.routing(T))
        err = case.check_outputs(x, out)
        print("  max rel err %.3e" % err, flush=True)
        # the streaming variant on the same inputs agrees on routing bit for bit
        other = GpuCase(cfg, seed=T + E, sched=_lib.SCHED_STREAM, inputs=case.inp)
        try:
            out2 = other.run()
            r1, r2 = case.launcher.routing(T), other.launcher.routing(T)
            assert np.array_equal(r1["topk_idx"], r2["topk_idx"])
            assert np.array_equal(r1["perm"], r2["perm"])
            # Outputs: the streaming variant sums float rows and rounds once; the tiled one
            # rounds each slot's down-projection row to bf16 first (relative 2^-9 each, the
            # weights sum to 1), then both round the sum to bf16. Per token the two may
            # therefore differ by a bf16 ulp or two (2^-7 relative) of the row's largest
            # element, and by no more.
            a, b = out.float(), out2.float()
            ulp = a.abs().max(dim=1, keepdim=True).values * 2.0 ** -7
            worst = float(((a - b).abs() / ulp).max())
            print("  tiled vs streaming: %.2f bf16 ulps of the row maximum" % worst, flush=True)
            assert worst <= 2.0          # measured: at most 1.00
        finally:
            other.close()
        # the tiled variant reading the packed weight copy computes the same bits
        packed = GpuCase(cfg, seed=T + E, sched=_lib.SCHED_TILED, inputs=case.inp, pack_weights=True)
        try:
            assert packed.launcher.sched_for(T) == _lib.SCHED_TILED
            assert torch.equal(packed.run(), out)
        finally:
            packed.close()
    finally:
        case.close()


@pytest.mark.parametrize("name,T", [("qwen3_30b_decode", 64), ("qwen3_30b_decode", 100),
                                    ("tiny_f32", 16)])
def test_packed_weights_equal_unpacked(name, T):
    """The packed second copy of the expert weights changes where bytes are read
    from, not what is computed."""
    cfg = synth.CONFIGS[name].replace(T=T)
    a = GpuCase(cfg, seed=11, sched=_lib.SCHED_STREAM)
    try:
        b = GpuCase(cfg, seed=11, sched=_lib.SCHED_STREAM, inputs=a.inp, pack_weights=True)
        try:
            out_a, out_b = a.run(), b.run()
            assert torch.equal(out_a, out_b)
            b.check_routing(b.inp["tokens"], b.launcher.routing(T))
            b.check_outputs(b.inp["tokens"], out_b, None if T <= 64 else np.arange(0, T, 7))
            # refresh after an in-place weight change
            b.inp["ffn2"].mul_(2.0)
            b.launcher.refresh_weights()
            a_out2, b_out2 = a.run(), b.run()
            assert torch.equal(a_out2, b_out2)
            b.inp["ffn2"].mul_(0.5)
        finally:
            b.close()
    finally:
        a.close()


@pytest.mark.parametrize("name,T,sched", [("qwen3_30b_decode", 64, _lib.SCHED_STREAM),
                                          ("qwen3_30b_decode", 700, _lib.SCHED_TILED),
                                          ("tiny_f32", 16, _lib.SCHED_STREAM),
                                          # several row tiles an expert: their tasks share the weights
                                          ("qwen3_30b_decode", 1500, _lib.SCHED_STREAM),
                                          ("tiny_f32", 600, _lib.SCHED_STREAM)])
def test_prepacked_weights_equal_unpacked(name, T, sched):
    """Weights packed in place by the caller (no second copy anywhere, the
    launcher's workspace holds no weight-sized region) give the same bits as the
    row-major tensors and as the launcher's own packed copy."""
    import ctypes

    cfg = synth.CONFIGS[name].replace(T=T)
    a = GpuCase(cfg, seed=11, sched=sched)
    try:
        out_a = a.run()
        packed_inp = dict(a.inp)
        packed_inp["ffn1"] = a.inp["ffn1"].clone()
        packed_inp["ffn2"] = a.inp["ffn2"].clone()
        a.launcher.pack_weights_in_place(packed_inp["ffn1"], packed_inp["ffn2"])
        torch.cuda.synchronize()
        assert not torch.equal(packed_inp["ffn1"], a.inp["ffn1"])     # it really is another layout
        b = GpuCase(cfg, seed=11, sched=sched, inputs=packed_inp, prepacked=True)
        try:
            assert torch.equal(b.run(), out_a)
            b.check_routing(b.inp["tokens"], b.launcher.routing(T))
            # workspace: nothing weight-sized
            d = _lib.LayerDesc()
            d.experts, d.hidden, d.intermediate, d.top_k = cfg.E, cfg.H, cfg.I, cfg.k
            d.dtype = _lib.BF16 if cfg.dtype == "bf16" else _lib.F32
            d.max_tokens, d.sched, d.flags = T, sched, _lib.FLAG_WEIGHTS_PREPACKED
            n_pre, n_copy = ctypes.c_size_t(0), ctypes.c_size_t(0)
            assert _lib.load().flashMoeWorkspaceBytes(ctypes.byref(d), ctypes.byref(n_pre)) == 0
            d.flags = _lib.FLAG_PACK_WEIGHTS
            assert _lib.load().flashMoeWorkspaceBytes(ctypes.byref(d), ctypes.byref(n_copy)) == 0
            esz = 2 if cfg.dtype == "bf16" else 4
            assert n_copy.value - n_pre.value >= 3 * cfg.E * cfg.H * cfg.I * esz
        finally:
            b.close()
        c = GpuCase(cfg, seed=11, sched=sched, inputs=a.inp, pack_weights=True)
        try:
            assert torch.equal(c.run(), out_a)
        finally:
            c.close()
    finally:
        a.close()
