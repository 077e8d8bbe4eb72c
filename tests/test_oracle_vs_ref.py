"""The restatement against the reference's own headers compiled in
oracle/_ref (present only where the reference checkout was available at build
time; skipped elsewhere — the golden vectors cover that case)."""
import numpy as np
import pytest

from flash_distributed_moe_amd import synth
from oracle import oracle

pytestmark = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built here")


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_whole_layer(seed):
    rng = np.random.default_rng(seed)
    E = int(rng.choice([4, 8, 24]))
    k = int(rng.integers(1, min(E, 8) + 1))
    cfg = synth.MoeConfig("r", int(rng.integers(1, 12)), int(rng.choice([32, 80, 192])), E, k,
                          int(rng.choice([8, 24, 56])), str(rng.choice(["f32", "bf16"])))
    inp = synth.make_inputs_np(cfg, seed=100 + seed)
    scale = np.float32(rng.choice([1.0, 25.0]))          # sharper routing / larger activations
    gate = inp["gate"] * scale
    out, idx, w = oracle.forward(inp["tokens"], gate, inp["ffn1"], inp["ffn2"], k)
    ridx, rw = oracle.ref_moe_gate(inp["tokens"], gate, k)
    rout = oracle.ref_full_moe(inp["tokens"], gate, inp["ffn1"], inp["ffn2"], k)
    assert np.array_equal(idx, ridx) and np.array_equal(w, rw) and np.array_equal(out, rout)


def test_gemm_topk_softmax_pieces():
    rng = np.random.default_rng(42)
    a = rng.standard_normal((9, 130)).astype(np.float32)
    b = rng.standard_normal((17, 130)).astype(np.float32)
    assert np.array_equal(oracle.logits(a, b), oracle.ref_gemm(a, b))
    m = rng.integers(-3, 4, size=(30, 17)).astype(np.float32)
    v, i = oracle.topk(m, 5)
    rv, ri = oracle.ref_topk(m, 5)
    assert np.array_equal(i, ri) and np.array_equal(v, rv)
    s = (rng.standard_normal((20, 8)) * 10).astype(np.float32)
    assert np.array_equal(oracle.softmax_rows(s), oracle.ref_softmax_rows(s))
