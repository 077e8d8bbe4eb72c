"""Shared helpers for the parity tests."""
import hashlib

import numpy as np


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return np.frombuffer(h.digest(), dtype=np.uint8).copy()


def dense_moe_f64(tokens, gate, ffn1, ffn2, topk_idx, topk_w):
    """Independent float64 restatement of the expert stage as dense algebra.

    out[t] = sum_s w[t,s] * W2[e] @ (silu(W1[e] @ x_t) * (W3[e] @ x_t)).
    """
    x = tokens.astype(np.float64)
    T, H = x.shape
    I = ffn2.shape[2]
    out = np.zeros((T, H))
    for t in range(T):
        for s in range(topk_idx.shape[1]):
            e = int(topk_idx[t, s])
            if e < 0:
                continue
            gu = ffn1[e].astype(np.float64) @ x[t]
            a, b = gu[:I], gu[I:]
            h = a / (1.0 + np.exp(-a)) * b
            out[t] += float(topk_w[t, s]) * (ffn2[e].astype(np.float64) @ h)
    return out


def max_rel_err(got, ref):
    """max|got-ref| / max|ref| — the relative-error measure used for outputs."""
    ref = np.asarray(ref, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    return float(np.max(np.abs(got - ref)) / max(np.max(np.abs(ref)), 1e-30))
