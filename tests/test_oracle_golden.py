"""The CPU oracle against the golden vectors written from the reference's own
CPU MoE headers (tests/golden/make_golden.py). Same compiler flags and libm on
both sides, so equality is exact."""
import os

import numpy as np
import pytest

from flash_distributed_moe_amd import synth
from oracle import oracle
from tests.golden.make_golden import SMALL_SHAPES
from tests.helpers import digest


def load(golden_dir, name):
    return np.load(os.path.join(golden_dir, name), allow_pickle=False)


def test_tiny_f32_whole_layer(golden_dir):
    g = load(golden_dir, "ref_tiny_f32.npz")
    cfg = synth.CONFIGS["tiny_f32"]
    inp = synth.make_inputs_np(cfg, seed=int(g["seed"]))
    assert np.array_equal(
        digest(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"]), g["input_digest"]
    ), "synthetic input generator drifted from the one the fixture was made with"
    out, idx, w = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], cfg.k)
    assert np.array_equal(idx, g["topk_idx"])
    assert np.array_equal(w, g["topk_w"])
    assert np.array_equal(out, g["out"])
    # thread count does not change a bit
    out1, _, _ = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], cfg.k,
                                nthreads=1)
    assert np.array_equal(out1, out)


@pytest.mark.parametrize("shape", SMALL_SHAPES, ids=[s[0] for s in SMALL_SHAPES])
def test_small_shapes(golden_dir, shape):
    g = load(golden_dir, "ref_small_shapes.npz")
    name, T, H, E, k, I, dt, seed = shape
    inp = synth.make_inputs_np(synth.MoeConfig(name, T, H, E, k, I, dt), seed=seed)
    assert np.array_equal(digest(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"]),
                          g[name + "_digest"])
    out, idx, w = oracle.forward(inp["tokens"], inp["gate"], inp["ffn1"], inp["ffn2"], k)
    assert np.array_equal(idx, g[name + "_idx"])
    assert np.array_equal(w, g[name + "_w"])
    assert np.array_equal(out, g[name + "_out"])


def test_gate_30b_shape(golden_dir):
    g = load(golden_dir, "ref_gate_30b.npz")
    c = synth.CONFIGS["qwen3_30b_decode"]
    gate = synth.normal_np(7907, synth.STREAM_GATE, (c.E, c.H), synth.SIGMA_W, True)
    x = synth.normal_np(7907, synth.STREAM_TOKENS, (32, c.H), synth.SIGMA_X, True)
    assert np.array_equal(digest(x, gate), g["input_digest"])
    idx, w = oracle.gate(x, gate, c.k)
    assert np.array_equal(idx, g["topk_idx"])
    assert np.array_equal(w, g["topk_w"])


def test_topk_ties_nan_short_rows(golden_dir):
    g = load(golden_dir, "ref_topk_softmax_cases.npz")
    v, i = oracle.topk(g["tie_rows"], 4)
    assert np.array_equal(i, g["tie_idx"])
    assert np.array_equal(v, g["tie_vals"], equal_nan=True)
    # ties by hand: {1,3,3,0,3,1,1,-2}, k=4 -> the three 3s in index order, then the first 1
    assert i[0].tolist() == [1, 2, 4, 0]
    v, i = oracle.topk(g["short_rows"], 5)
    assert np.array_equal(i, g["short_idx"])
    assert np.array_equal(v, g["short_vals"])
    assert i[0].tolist() == [1, 0, 2, -1, -1]


def test_softmax_rows(golden_dir):
    g = load(golden_dir, "ref_topk_softmax_cases.npz")
    assert np.array_equal(oracle.softmax_rows(g["softmax_in"]), g["softmax_out"])


def test_reference_rand_recipe(golden_dir):
    g = load(golden_dir, "ref_rand_inputs_small.npz")
    T, E, H, I, k = (int(g[n]) for n in "TEHIk")
    tok, gw, f1, f2 = oracle.reference_test_inputs(T, E, H, I, seed=7907)
    assert np.array_equal(digest(tok, gw, f1, f2), g["input_digest"])
    assert tok.min() >= -1 and tok.max() <= 1 and np.abs(gw).max() <= np.float32(0.1)
    out, _, _ = oracle.forward(tok, gw, f1, f2, k)
    assert np.array_equal(out, g["out"])


def test_ffn1_stage(golden_dir):
    g = load(golden_dir, "ref_ffn1.npz")
    c = synth.MoeConfig("ffn1", 4, 64, 1, 1, 24, "f32")
    inp = synth.make_inputs_np(c, seed=int(g["seed"]))
    x = inp["tokens"] * np.float32(40.0)
    w13 = inp["ffn1"][0] * np.float32(20.0)
    # expert stage with one expert, weight 1 and an identity down projection
    eye = np.zeros((1, c.H, c.I), np.float32)           # down-proj [E,H,I]: identity block
    eye[0, :c.I, :] = np.eye(c.I, dtype=np.float32)
    idx = np.zeros((4, 1), np.int32)
    w = np.ones((4, 1), np.float32)
    got = oracle.experts(x, w13[None], eye, idx, w)
    assert np.array_equal(got[:, :c.I], g["out"])
    assert np.all(got[:, c.I:] == 0)
