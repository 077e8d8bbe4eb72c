"""Pins the CPU oracle against what the mathematics fixes, independently of the
reference: float64 algebra, closed forms, exact integer cases and brute force.
Each check is chosen so that a plausible slip (transposed operand, wrong tie
rule, softmax over all experts instead of the winners, missing gate weight,
gate/up halves swapped) fails it."""
import itertools

import numpy as np
import pytest

from flash_distributed_moe_amd import synth
from oracle import oracle
from tests.helpers import dense_moe_f64, max_rel_err


def test_logits_exact_on_small_integers():
    # small integers: every partial sum is exact in float32, so any summation
    # order gives the same bits and int64 numpy is the truth
    rng = np.random.default_rng(0)
    x = rng.integers(-8, 9, size=(5, 37)).astype(np.float32)
    g = rng.integers(-8, 9, size=(11, 37)).astype(np.float32)
    b = rng.integers(-3, 4, size=11).astype(np.float32)
    want = x.astype(np.int64) @ g.astype(np.int64).T + b.astype(np.int64)
    assert np.array_equal(oracle.logits(x, g, b), want.astype(np.float32))
    assert oracle.logits(x, g).shape == (5, 11)          # [T,E], not [E,T]


def test_logits_sequential_order_differs_from_pairwise():
    # the oracle adds products one by one in ascending k; a hand-rolled float32
    # loop is the definition
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 300)).astype(np.float32)
    g = rng.standard_normal((3, 300)).astype(np.float32)
    want = np.zeros((2, 3), np.float32)
    for t in range(2):
        for e in range(3):
            acc = np.float32(0)
            for k in range(300):
                acc = np.float32(acc + np.float32(x[t, k] * g[e, k]))
            want[t, e] = acc
    assert np.array_equal(oracle.logits(x, g), want)
    assert np.allclose(want, x.astype(np.float64) @ g.astype(np.float64).T, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("seed", range(5))
def test_topk_is_stable_argsort(seed):
    rng = np.random.default_rng(seed)
    m = rng.integers(-4, 5, size=(40, 24)).astype(np.float32)   # many ties
    vals, idx = oracle.topk(m, 6)
    order = np.argsort(-m, axis=1, kind="stable")[:, :6]
    assert np.array_equal(idx, order)
    assert np.array_equal(vals, np.take_along_axis(m, order, 1))


def test_topk_brute_force_tiny():
    # all 3^4 rows over {0,1,2}: winners are the lexicographically first
    # positions among equal values
    for row in itertools.product([0.0, 1.0, 2.0], repeat=4):
        _, idx = oracle.topk(np.array([row], np.float32), 2)
        want = sorted(range(4), key=lambda c: (-row[c], c))[:2]
        assert idx[0].tolist() == want


def test_gate_weights_are_softmax_over_winners_only():
    cfg = synth.MoeConfig("g", 12, 64, 16, 4, 8, "f32")
    inp = synth.make_inputs_np(cfg, seed=3)
    x, g = inp["tokens"], inp["gate"] * np.float32(30.0)
    idx, w, lg = oracle.gate(x, g, 4, want_logits=True)
    win = np.take_along_axis(lg, idx, 1).astype(np.float64)
    sm = np.exp(win - win.max(1, keepdims=True))
    sm /= sm.sum(1, keepdims=True)
    assert np.allclose(w, sm, rtol=1e-6, atol=1e-7)
    assert np.allclose(w.sum(1), 1.0, atol=1e-6)
    assert np.all(np.diff(w, axis=1) <= 0)                # descending weights
    # equals full softmax -> top-k -> renormalise (Qwen3 norm_topk_prob)
    full = np.exp(lg.astype(np.float64) - lg.max(1, keepdims=True))
    full /= full.sum(1, keepdims=True)
    top = np.take_along_axis(full, idx, 1)
    assert np.allclose(w, top / top.sum(1, keepdims=True), rtol=1e-6)
    # and is NOT the un-renormalised full softmax
    assert not np.allclose(w, top, rtol=1e-3)


def test_router_bias_shifts_selection():
    cfg = synth.MoeConfig("b", 64, 128, 16, 2, 8, "f32")
    inp = synth.make_inputs_np(cfg, seed=5)
    bias = np.zeros(16, np.float32)
    bias[[3, 9]] = 100.0
    idx, _ = oracle.gate(inp["tokens"], inp["gate"], 2, bias=bias)
    assert np.all(np.sort(idx, axis=1) == np.array([3, 9]))
    idx0, w0 = oracle.gate(inp["tokens"], inp["gate"], 2, bias=np.zeros(16, np.float32))
    idx1, w1 = oracle.gate(inp["tokens"], inp["gate"], 2)
    assert np.array_equal(idx0, idx1) and np.array_equal(w0, w1)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_forward_matches_dense_float64(dt):
    cfg = synth.MoeConfig("d", 10, 96, 12, 3, 40, dt)
    inp = synth.make_inputs_np(cfg, seed=17)
    out, idx, w = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], cfg.k)
    want = dense_moe_f64(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], idx, w)
    assert max_rel_err(out, want) < 2e-6
    # swapping the gate and up halves must be visible
    swapped = np.concatenate([inp["ffn1"][:, cfg.I:], inp["ffn1"][:, :cfg.I]], axis=1)
    wrong = dense_moe_f64(inp["tokens"], inp["gate"], swapped, inp["ffn2"], idx, w)
    assert max_rel_err(out, wrong) > 1e-2


def test_forward_linearity_in_down_projection():
    cfg = synth.MoeConfig("l", 6, 64, 8, 2, 32, "f32")
    inp = synth.make_inputs_np(cfg, seed=23)
    a, _, _ = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], 2)
    b, _, _ = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"] * np.float32(2),
                             2)
    assert np.array_equal(b, a * np.float32(2))           # power of two: exact


def test_permute_is_stable_sort_by_expert():
    rng = np.random.default_rng(7)
    T, E, k = 50, 12, 4
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    counts, offsets, perm = oracle.permute(idx, E)
    flat = idx.reshape(-1)
    assert np.array_equal(perm, np.argsort(flat, kind="stable"))
    assert np.array_equal(counts, np.bincount(flat, minlength=E))
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))
    # inside one expert the token ids ascend
    for e in range(E):
        seg = perm[offsets[e]:offsets[e + 1]] // k
        assert np.all(np.diff(seg) > 0)


def test_permute_drops_unfilled_slots():
    idx = np.array([[2, -1], [0, 2], [-1, -1]], np.int32)
    counts, offsets, perm = oracle.permute(idx, 3)
    assert counts.tolist() == [1, 0, 2] and perm.tolist() == [2, 0, 3]


def test_synth_numpy_and_torch_agree():
    import torch

    a = synth.normal_np(9, 2, (33, 65), 0.02, bf16=True)
    b = synth.normal_torch(9, 2, (33, 65), 0.02, torch.bfloat16, "cpu").float().numpy()
    assert np.array_equal(a, b)
    a = synth.normal_np(9, 4, (7, 129), 1.0)
    b = synth.normal_torch(9, 4, (7, 129), 1.0, torch.float32, "cpu").numpy()
    assert np.array_equal(a, b)
    assert abs(a.std() - 1) < 0.1 and abs(a.mean()) < 0.1
    # bf16 rounding matches torch's round-to-nearest-even
    r = np.random.default_rng(0).standard_normal(10000).astype(np.float32)
    assert np.array_equal(synth.bf16_round_np(r),
                          torch.from_numpy(r).to(torch.bfloat16).float().numpy())


def test_rmsnorm_closed_forms():
    # a constant row a with eps = 16 - a^2: mean + eps = 16, scale = 1/4 exactly, so
    # xn = a/4 * weight in exact arithmetic. eps added to the sum instead of the mean,
    # or to the root instead of the mean square, gives something else.
    H = 64
    w = np.linspace(-2, 2, H).astype(np.float32)
    x = np.full((1, H), 3.0, np.float32)
    assert np.array_equal(oracle.rmsnorm(x, w, 7.0), (0.75 * w)[None, :])
    # one-hot row of height v: mean = v^2/H, scale = sqrt(H)/|v| = 8/|v|
    x = np.zeros((1, H), np.float32)
    x[0, 5] = -4.0
    want = np.zeros((1, H), np.float32)
    want[0, 5] = -8.0 * w[5]
    assert np.array_equal(oracle.rmsnorm(x, w, 0.0), want)


def test_rmsnorm_against_float64_and_invariants():
    rng = np.random.default_rng(3)
    T, H = 9, 320
    x = (rng.standard_normal((T, H)) * rng.uniform(0.01, 30, (T, 1))).astype(np.float32)
    w = rng.uniform(0.5, 1.5, H).astype(np.float32)
    eps = 1e-6
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w
    got = oracle.rmsnorm(x, w, eps)
    assert got.dtype == np.float32 and np.max(np.abs(got - want) / np.abs(want)) < 3e-7
    # weight 1, eps 0: every row comes out with unit mean square
    unit = oracle.rmsnorm(x, np.ones(H, np.float32), 0.0).astype(np.float64)
    assert np.allclose((unit ** 2).mean(axis=1), 1.0, atol=1e-6)
    # a power of two on the input cancels exactly (eps = 0)
    assert np.array_equal(oracle.rmsnorm(x * np.float32(8), w, 0.0), oracle.rmsnorm(x, w, 0.0))
    # bf16: the nearest bfloat16 (ties to even) of the float32 result
    import torch

    rounded = oracle.rmsnorm(x, w, eps, bf16=True)
    assert np.array_equal(rounded, torch.from_numpy(got).to(torch.bfloat16).float().numpy())


def test_layer_edges_reduce_and_compose():
    cfg = synth.MoeConfig("edges", 12, 64, 8, 2, 32, "f32")
    inp = synth.make_inputs_np(cfg, 11)
    args = (inp["gate"], inp["ffn1"], inp["ffn2"], cfg.k)
    base, idx, wts = oracle.forward(inp["tokens"], *args)
    plain = oracle.layer(inp["tokens"], *args)
    assert np.array_equal(plain[0], base) and np.array_equal(plain[1], idx)
    # zero down projection: the layer contributes nothing, the residual is the input itself
    zero = (inp["gate"], inp["ffn1"], np.zeros_like(inp["ffn2"]), cfg.k)
    assert np.array_equal(oracle.layer(inp["tokens"], *zero, residual=True)[0], inp["tokens"])
    # the residual is the un-normalised row, and it is added once
    g = np.linspace(0.5, 1.5, cfg.H).astype(np.float32)
    both = oracle.layer(inp["tokens"], *args, norm_weight=g, norm_eps=0.0, residual=True)[0]
    normed = oracle.layer(inp["tokens"], *args, norm_weight=g, norm_eps=0.0)[0]
    assert np.allclose(both - normed, inp["tokens"], atol=1e-6)
    # with the norm in front the layer no longer sees the input's scale, without it it does
    big = inp["tokens"] * np.float32(4)
    assert np.array_equal(oracle.layer(big, *args, norm_weight=g, norm_eps=0.0)[0], normed)
    assert not np.array_equal(oracle.layer(big, *args)[0], base)
    # and it sees the normalised rows: the same as handing those rows to forward()
    assert np.array_equal(normed, oracle.forward(oracle.rmsnorm(inp["tokens"], g, 0.0), *args)[0])
