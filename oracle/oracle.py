"""TEST INFRASTRUCTURE ONLY: ctypes loader for the CPU oracle.

Wraps ``libmoe_oracle.so`` (the restatement of the reference's CPU MoE,
``moe_oracle.cpp``) and, where it has been built, ``_ref/libref_moe.so`` (the
reference's own headers compiled behind C entry points). Only tests, the smoke
check and the benchmark's cpu_baseline leg may import this module; the product
path never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_moe.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int)


def build(ref=False):
    """Compile the oracle (and the reference headers when ``ref``)."""
    targets = ["all"] + (["ref"] if ref else [])
    subprocess.check_call(["make", "-C", _HERE, "-B"] + targets)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_i32p)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def have_ref():
    return os.path.exists(_REF_PATH)


def ref():
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(_REF_PATH)
    return _ref


def default_threads():
    return max(1, min(16, os.cpu_count() or 1))


# ----------------------------------------------------------------- restatement
def logits(tokens, gate, bias=None, nthreads=None):
    tokens, tp = _f32(tokens)
    gate, gp = _f32(gate)
    T, H = tokens.shape
    E = gate.shape[0]
    assert gate.shape[1] == H
    bp = None
    if bias is not None:
        bias, bp = _f32(bias)
    out = np.empty((T, E), np.float32)
    lib().oracle_logits(tp, gp, bp, T, E, H, out.ctypes.data_as(_f32p),
                        nthreads or default_threads())
    return out


def topk(matrix, k):
    matrix, mp = _f32(matrix)
    rows, cols = matrix.shape
    vals = np.empty((rows, k), np.float32)
    idx = np.empty((rows, k), np.int32)
    lib().oracle_topk(mp, rows, cols, k, vals.ctypes.data_as(_f32p),
                      idx.ctypes.data_as(_i32p))
    return vals, idx


def softmax_rows(matrix):
    m = np.array(matrix, dtype=np.float32, order="C", copy=True)
    rows, cols = m.shape
    lib().oracle_softmax_rows(m.ctypes.data_as(_f32p), rows, cols)
    return m


def gate(tokens, gate_w, k, bias=None, want_logits=False, nthreads=None):
    tokens, tp = _f32(tokens)
    gate_w, gp = _f32(gate_w)
    T, H = tokens.shape
    E = gate_w.shape[0]
    bp = None
    if bias is not None:
        bias, bp = _f32(bias)
    lg = np.empty((T, E), np.float32) if want_logits else None
    idx = np.empty((T, k), np.int32)
    w = np.empty((T, k), np.float32)
    lib().oracle_gate(tp, gp, bp, T, E, H, k,
                      lg.ctypes.data_as(_f32p) if want_logits else None,
                      idx.ctypes.data_as(_i32p), w.ctypes.data_as(_f32p),
                      nthreads or default_threads())
    return (idx, w, lg) if want_logits else (idx, w)


def permute(topk_idx, E):
    topk_idx, ip = _i32(topk_idx)
    T, k = topk_idx.shape
    counts = np.empty(E, np.int32)
    offsets = np.empty(E + 1, np.int32)
    perm = np.full(T * k, -1, np.int32)
    n = lib().oracle_permute(ip, T, E, k, counts.ctypes.data_as(_i32p),
                             offsets.ctypes.data_as(_i32p),
                             perm.ctypes.data_as(_i32p))
    return counts, offsets, perm[:n]


def forward(tokens, gate_w, ffn1, ffn2, k, bias=None, nthreads=None):
    """Returns (out[T,H], topk_idx[T,k], topk_w[T,k])."""
    tokens, tp = _f32(tokens)
    gate_w, gp = _f32(gate_w)
    ffn1, f1p = _f32(ffn1)
    ffn2, f2p = _f32(ffn2)
    T, H = tokens.shape
    E = gate_w.shape[0]
    I = ffn2.shape[2]
    assert ffn1.shape == (E, 2 * I, H) and ffn2.shape == (E, H, I)
    bp = None
    if bias is not None:
        bias, bp = _f32(bias)
    out = np.empty((T, H), np.float32)
    idx = np.empty((T, k), np.int32)
    w = np.empty((T, k), np.float32)
    lib().oracle_forward(tp, gp, f1p, f2p, bp, T, E, H, k, I,
                         out.ctypes.data_as(_f32p), idx.ctypes.data_as(_i32p),
                         w.ctypes.data_as(_f32p), nthreads or default_threads())
    return out, idx, w


def _round_bf16(a):
    """float32 -> nearest-even bfloat16, kept as float32."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def rmsnorm(tokens, weight, eps, bf16=False):
    """xn[t,k] = (x[t,k] * float32(1 / sqrt(mean_k x[t,k]^2 + eps))) * weight[k]: mean, sqrt
    and reciprocal in float64, the two products in float32, and for bf16=True one rounding
    to bfloat16. Not part of the reference's layer (refFullMoe.h:9-70 starts at the gate):
    it is the definition the library's optional FLASH_MOE_FLAG_RMSNORM step is held to,
    the usual RMSNorm (x / rms(x) * weight) with the roundings spelled out. Pinned in
    tests/test_oracle_math.py against float64 algebra (unit-RMS rows under weight 1,
    scale invariance, a closed-form row), not against a reference vector."""
    x = np.ascontiguousarray(tokens, np.float32)
    w = np.ascontiguousarray(weight, np.float32)
    ss = np.einsum("tk,tk->t", x.astype(np.float64), x.astype(np.float64))
    scale = (1.0 / np.sqrt(ss / np.float64(x.shape[1]) + np.float64(eps))).astype(np.float32)
    xn = (x * scale[:, None]) * w[None, :]
    return _round_bf16(xn) if bf16 else xn


def layer(tokens, gate_w, ffn1, ffn2, k, bias=None, norm_weight=None, norm_eps=1e-6, residual=False,
          bf16=False, nthreads=None):
    """forward() with the two optional steps at its edges: the layer runs on
    rmsnorm(tokens) when norm_weight is given, and the input rows are added to its output
    (one float32 addition per element) when residual is set. With neither it is forward()."""
    x = np.ascontiguousarray(tokens, np.float32)
    xin = x if norm_weight is None else rmsnorm(x, norm_weight, norm_eps, bf16)
    out, idx, w = forward(xin, gate_w, ffn1, ffn2, k, bias, nthreads)
    if residual:
        out = out + x
    return out, idx, w


def experts(tokens, ffn1, ffn2, topk_idx, topk_w, nthreads=None):
    tokens, tp = _f32(tokens)
    ffn1, f1p = _f32(ffn1)
    ffn2, f2p = _f32(ffn2)
    topk_idx, ip = _i32(topk_idx)
    topk_w, wp = _f32(topk_w)
    T, H = tokens.shape
    E, _, I = ffn2.shape
    k = topk_idx.shape[1]
    out = np.empty((T, H), np.float32)
    lib().oracle_experts(tp, f1p, f2p, T, E, H, k, I, ip, wp,
                         out.ctypes.data_as(_f32p), nthreads or default_threads())
    return out


def reference_test_inputs(T, E, H, I, seed=7907):
    """Inputs as the reference's own tests draw them (glibc rand())."""
    tokens = np.empty((T, H), np.float32)
    gate_w = np.empty((E, H), np.float32)
    ffn1 = np.empty((E, 2 * I, H), np.float32)
    ffn2 = np.empty((E, H, I), np.float32)
    fn = lib().oracle_reference_test_inputs
    fn.argtypes = [ctypes.c_uint, _f32p, ctypes.c_size_t, _f32p, ctypes.c_size_t,
                   _f32p, ctypes.c_size_t, _f32p, ctypes.c_size_t]
    fn(seed, tokens.ctypes.data_as(_f32p), tokens.size,
       gate_w.ctypes.data_as(_f32p), gate_w.size,
       ffn1.ctypes.data_as(_f32p), ffn1.size,
       ffn2.ctypes.data_as(_f32p), ffn2.size)
    return tokens, gate_w, ffn1, ffn2


# ------------------------------------------------- compiled reference headers
def ref_gemm(a, b):
    a, ap = _f32(a)
    b, bp = _f32(b)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), np.float32)
    ref().ref_gemm(ap, bp, m, n, k, c.ctypes.data_as(_f32p))
    return c


def ref_topk(matrix, k):
    matrix, mp = _f32(matrix)
    rows, cols = matrix.shape
    vals = np.empty((rows, k), np.float32)
    idx = np.empty((rows, k), np.int32)
    ref().ref_topk(mp, rows, cols, k, vals.ctypes.data_as(_f32p),
                   idx.ctypes.data_as(_i32p))
    return vals, idx


def ref_softmax_rows(matrix):
    m = np.array(matrix, dtype=np.float32, order="C", copy=True)
    ref().ref_softmax_rows(m.ctypes.data_as(_f32p), m.shape[0], m.shape[1])
    return m


def ref_moe_gate(tokens, gate_w, k):
    tokens, tp = _f32(tokens)
    gate_w, gp = _f32(gate_w)
    T, H = tokens.shape
    E = gate_w.shape[0]
    w = np.empty((T, k), np.float32)
    idx = np.empty((T, k), np.int32)
    ref().ref_moe_gate(tp, gp, T, E, H, k, w.ctypes.data_as(_f32p),
                       idx.ctypes.data_as(_i32p))
    return idx, w


def ref_expert_ffn1(tokens, w13):
    tokens, tp = _f32(tokens)
    w13, wp = _f32(w13)
    T, H = tokens.shape
    I = w13.shape[0] // 2
    out = np.empty((T, I), np.float32)
    ref().ref_expert_ffn1(tp, wp, T, H, I, out.ctypes.data_as(_f32p))
    return out


def ref_full_moe(tokens, gate_w, ffn1, ffn2, k):
    tokens, tp = _f32(tokens)
    gate_w, gp = _f32(gate_w)
    ffn1, f1p = _f32(ffn1)
    ffn2, f2p = _f32(ffn2)
    T, H = tokens.shape
    E = gate_w.shape[0]
    I = ffn2.shape[2]
    out = np.empty((T, H), np.float32)
    ref().ref_full_moe(tp, gp, f1p, f2p, T, E, H, k, I,
                       out.ctypes.data_as(_f32p))
    return out
