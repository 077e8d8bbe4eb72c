"""Behaviour at the launcher boundary on the GPU: empty and oversized batches,
the Python surface's checks, non-finite inputs, and the device-side time-out path
(forced from the host with a tiny wait limit; the kernel still exits normally)."""
import numpy as np
import pytest
import torch

from flash_distributed_moe_amd import synth
from oracle import oracle
from tests.helpers import max_rel_err
from tests.moe_case import GpuCase

pytestmark = pytest.mark.gpu

HIP_ERROR_UNKNOWN = 999


def test_empty_batch_is_a_no_op():
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=8, name="empty")
    case = GpuCase(cfg)
    try:
        x = case.inp["tokens"][:0]
        out = torch.empty_like(x)
        case.launcher.launch(x, out)
        torch.cuda.synchronize()
        assert case.launcher.status()[0] == 0
        # and the launcher still works afterwards
        got = case.run()
        case.check_outputs(case.inp["tokens"], got)
    finally:
        case.close()


def test_more_tokens_than_max_tokens_is_refused(capfd):
    cfg = synth.CONFIGS["qwen3_30b_decode"].replace(T=8, name="oversized")
    case = GpuCase(cfg)
    try:
        big = torch.cat([case.inp["tokens"], case.inp["tokens"]], 0)
        with pytest.raises(RuntimeError, match="hipError_t %d" % HIP_ERROR_UNKNOWN):
            case.launcher.launch(big, torch.empty_like(big))
        assert "exceeds max_tokens" in capfd.readouterr().out
    finally:
        case.close()


def test_python_surface_checks():
    cfg = synth.CONFIGS["tiny_f32"]
    case = GpuCase(cfg)
    try:
        x = case.inp["tokens"]
        with pytest.raises(RuntimeError, match="must be contiguous"):
            case.launcher.launch(x.t().contiguous().t(), torch.empty_like(x))
        with pytest.raises(RuntimeError, match="output shape must equal tokens shape"):
            case.launcher.launch(x, torch.empty_like(x[:-1]))
        with pytest.raises(RuntimeError, match="must be float32 or bfloat16"):
            case.launcher.launch(x.to(torch.bfloat16), torch.empty_like(x, dtype=torch.bfloat16))
        with pytest.raises(RuntimeError, match="CUDA tensor"):
            case.launcher.launch(x.cpu(), torch.empty_like(x.cpu()))
        assert case.launcher.valid
        case.launcher.destroy()
        assert not case.launcher.valid
        with pytest.raises(RuntimeError, match="Launcher was destroyed"):
            case.launcher.launch(x, torch.empty_like(x))
    finally:
        case.close()


@pytest.mark.parametrize("name", ["tiny_f32", "qwen3_30b_decode"])
def test_nan_and_all_equal_logits(name):
    """A token row of NaNs selects nothing (every slot -1, output row 0), a row of
    zeros makes every logit equal and must pick experts 0..k-1 in that order
    (refTopk.h:36-58: strict '>' keeps the first of equals)."""
    cfg = synth.CONFIGS[name].replace(T=6, name="nonfinite")
    case = GpuCase(cfg)
    try:
        x = case.inp["tokens"].clone()
        x[1] = float("nan")
        x[4] = 0.0
        out = torch.empty_like(x)
        case.launcher.launch(x, out)
        torch.cuda.synchronize()
        assert case.launcher.status()[0] == 0
        r = case.launcher.routing(cfg.T)
        assert (r["topk_idx"][1] == -1).all()
        assert list(r["topk_idx"][4]) == list(range(cfg.k))
        case.check_routing(x, r)
        got = out.float().cpu().numpy()
        assert (got[1] == 0).all() and (got[4] == 0).all()
        keep = [0, 2, 3, 5]
        hw = case.host_weights()
        ref, _, _ = oracle.forward(x.float().cpu().numpy()[keep], hw["gate"], hw["ffn1"], hw["ffn2"],
                                   cfg.k)
        tol = 1e-2 if cfg.dtype == "bf16" else 2e-5
        assert max_rel_err(got[keep], ref) <= tol
    finally:
        case.close()


@pytest.mark.parametrize("name,T,sched", [("qwen3_30b_decode", 64, 1), ("qwen3_30b_decode", 512, 2)])
def test_device_wait_limit_is_reported_and_cleared(name, T, sched):
    """With a wait limit of 100 ns every dependency wait that has to wait at all
    gives up: the kernel ends normally with NaN in its output, flashMoeStatus
    reports bit 1, and the next launch with the normal limit is correct again."""
    cfg = synth.CONFIGS[name].replace(T=T, name="timeout")
    case = GpuCase(cfg, sched=sched)
    try:
        x = case.inp["tokens"]
        good = case.run().clone()
        case.launcher.set_wait_limit_ms(1e-4)
        out = torch.zeros_like(x)
        case.launcher.launch(x, out)
        torch.cuda.synchronize()
        assert bool(torch.isnan(out).all()), "a failed launch must leave NaN in every output element"
        err, _ = case.launcher.status()
        assert err & 1, "the shortened wait did not time out"
        assert case.launcher.status()[0] == 0, "status must clear the error"
        case.launcher.set_wait_limit_ms(2000.0)
        again = case.run()
        assert torch.equal(again, good)
        case.check_outputs(x, again)
    finally:
        case.close()


@pytest.mark.parametrize("name,T,sched", [("qwen3_30b_decode", 64, 1),
                                          ("qwen3_30b_decode", 700, 2)])
def test_device_failure_reaches_a_caller_that_never_asks(name, T, sched, capfd):
    """A caller written against the reference's interface only ever calls Launch:
    after a launch has failed on the device, the next Launch returns
    hipErrorUnknown (nothing is launched), and the one after that is correct,
    with no call of flashMoeStatus in between. A captured graph keeps working too."""
    cfg = synth.CONFIGS[name].replace(T=T, name="timeout")
    case = GpuCase(cfg, sched=sched)
    try:
        x = case.inp["tokens"]
        good = case.run().clone()
        case.launcher.set_wait_limit_ms(1e-4)
        out = torch.zeros_like(x)
        case.launcher.launch(x, out)            # fails on the device; Launch itself has returned success
        torch.cuda.synchronize()
        case.launcher.set_wait_limit_ms(2000.0)
        untouched = torch.full_like(x, 3.0)
        with pytest.raises(RuntimeError, match="hipError_t 999"):
            case.launcher.launch(x, untouched)
        torch.cuda.synchronize()
        assert "an earlier launch failed on the device" in capfd.readouterr().out
        assert bool((untouched == 3.0).all())   # nothing was launched
        again = torch.empty_like(x)
        case.launcher.launch(x, again)          # the launcher re-armed itself on the device
        torch.cuda.synchronize()
        assert torch.equal(again, good)
        assert case.launcher.status()[0] & 1    # the bits are still there for whoever asks
        assert case.launcher.status()[0] == 0
    finally:
        case.close()


@pytest.mark.parametrize("shape", [
    # T, H, E, k, I, dtype, sched
    (24, 64, 4, 2, 32, "f32", 1),
    (40, 128, 8, 2, 64, "bf16", 1),
    (300, 256, 8, 2, 128, "bf16", 2),     # the tiled variant's gate/up tiles
])
def test_gate_up_stage_alone(shape):
    """The gate/up + SwiGLU stage by itself, as the reference tests it
    (test/singleGPU/cpp/moe/internal/moeExpertFFN1Test.hip:58-106, abs 1e-4 in
    float32): h read back from the device against the oracle's expert stage run
    with an identity down projection and weight 1, row by permuted row. (The
    golden vector written from the reference's refExpertFFN1, tests/golden/ref_ffn1.npz,
    has I = 24, which the launcher does not admit; it pins the oracle function used here.)"""
    T, H, E, k, I, dt, sched = shape
    cfg = synth.MoeConfig("ffn1", T, H, E, k, I, dt)
    case = GpuCase(cfg, seed=T + I, sched=sched)
    try:
        case.run()
        r = case.launcher.routing(T)
        h = case.launcher.intermediate(T)
        hw = case.host_weights()
        x = case.inp["tokens"].float().cpu().numpy()
        eye = np.zeros((1, H, I), np.float32)
        eye[0, :I, :] = np.eye(I, dtype=np.float32)
        one_idx, one_w = np.zeros((1, 1), np.int32), np.ones((1, 1), np.float32)
        worst = 0.0
        for row, entry in enumerate(r["perm"]):
            t, s = divmod(int(entry), k)
            e = int(r["topk_idx"][t, s])
            want = oracle.experts(x[t:t + 1], hw["ffn1"][e][None], eye, one_idx, one_w)[0, :I]
            tol = 1e-4 if dt == "f32" else 1e-2 * max(np.abs(want).max(), 1e-6)
            worst = max(worst, float(np.abs(h[row] - want).max() / (tol if dt == "f32" else 1.0)))
            assert np.allclose(h[row], want, rtol=0 if dt == "f32" else 8e-3, atol=tol), (row, t, s, e)
        print("  gate/up stage: %d rows checked" % len(r["perm"]), flush=True)
    finally:
        case.close()


@pytest.mark.parametrize("shape", [
    # T, H, E, k, I, dtype, sched
    (24, 64, 4, 2, 32, "f32", 1),
    (40, 128, 8, 2, 64, "bf16", 1),
    (300, 256, 8, 2, 128, "bf16", 2),     # the tiled variant: bf16 rows, weight applied by the combine step
    (700, 512, 4, 2, 256, "bf16", 2),     # the tiled variant on packed weights (register-staged pipeline)
])
def test_down_stage_alone(shape):
    """The down projection and its scaling by themselves, as the reference tests its expert
    stages apart from the sum over slots
    (test/singleGPU/cpp/moe/internal/moeExpertsTests.hip:389-475): the rows the combine step
    reads, copied back from the device, against the oracle's expert stage for that one
    (token, slot) alone: with the slot's gate weight where the variant keeps weighted rows,
    with weight 1 where it keeps them unweighted."""
    T, H, E, k, I, dt, sched = shape
    cfg = synth.MoeConfig("ffn2", T, H, E, k, I, dt)
    case = GpuCase(cfg, seed=T + H, sched=sched, pack_weights=(H == 512))
    try:
        case.run()
        r = case.launcher.routing(T)
        y, weighted = case.launcher.down_rows(T)
        assert weighted == (sched == 1)
        hw = case.host_weights()
        x = case.inp["tokens"].float().cpu().numpy()
        one_idx = np.zeros((1, 1), np.int32)
        checked = 0
        for t in range(0, T, 1 if T <= 64 else 7):
            for s in range(k):
                e = int(r["topk_idx"][t, s])
                w = np.full((1, 1), r["topk_w"][t, s] if weighted else 1.0, np.float32)
                want = oracle.experts(x[t:t + 1], hw["ffn1"][e][None], hw["ffn2"][e][None], one_idx, w)[0]
                got = y[t * k + s]
                scale = max(float(np.abs(want).max()), 1e-12)
                tol = 2e-5 if dt == "f32" else 1e-2
                assert float(np.abs(got - want).max()) <= tol * scale, (t, s, e)
                checked += 1
        print("  down stage: %d rows checked, %s" % (checked, "weighted float rows" if weighted else "unweighted bf16 rows"),
              flush=True)
    finally:
        case.close()
