"""Deterministic synthetic inputs for the MoE layer.

Values are approximately normal, built from integer arithmetic only so that
numpy on the CPU and torch on the CPU or GPU produce the same bits:

    h_j = mix64(base(seed, stream) + (3*i + j) * GOLDEN),  j = 0, 1, 2
    S   = sum of the twelve 16-bit fields of h_0, h_1, h_2     (Irwin-Hall, n=12)
    z   = (S - 6*65535) / 65536            exact in float32, mean 0, sd 1 (to 1e-9)
    v   = float32(z) * float32(sigma)      one IEEE multiply
    bf16 configs: v rounded to nearest-even bfloat16

``i`` is the flat index of the element in storage layout, so a token row is
the same whatever the batch size. Streams: 1 router weight [E,H], 2 gate/up
weight [E,2I,H], 3 down weight [E,H,I], 4 tokens [T,H], 5 hot-expert choice.
The tails stop at +-6 sigma; the router logits are sums of H products and are
Gaussian by the central limit theorem either way.
"""
import numpy as np

_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_C1 = 0xBF58476D1CE4E5B9
_C2 = 0x94D049BB133111EB

STREAM_GATE, STREAM_FFN1, STREAM_FFN2, STREAM_TOKENS, STREAM_HOT = 1, 2, 3, 4, 5


def _mix64_int(z):
    z &= _M64
    z = ((z ^ (z >> 30)) * _C1) & _M64
    z = ((z ^ (z >> 27)) * _C2) & _M64
    return z ^ (z >> 31)


def stream_base(seed, stream):
    return _mix64_int((int(seed) * 0x100000001B3 + int(stream)) & _M64)


def _mix64_np(z):
    z = (z ^ (z >> np.uint64(30))) * np.uint64(_C1)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(_C2)
    return z ^ (z >> np.uint64(31))


def irwin_hall_np(seed, stream, start, count):
    """float32 z-values for flat indices [start, start+count) (numpy)."""
    base = np.uint64(stream_base(seed, stream))
    i = np.arange(start, start + count, dtype=np.uint64)
    s = np.zeros(count, dtype=np.int64)
    with np.errstate(over="ignore"):
        for j in range(3):
            h = _mix64_np(base + (i * np.uint64(3) + np.uint64(j)) * np.uint64(_GOLDEN))
            for f in range(4):
                s += ((h >> np.uint64(16 * f)) & np.uint64(0xFFFF)).astype(np.int64)
    return ((s - 6 * 65535).astype(np.float32)) / np.float32(65536.0)


def bf16_round_np(x):
    """Round float32 to the nearest-even bfloat16, returned as float32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


def normal_np(seed, stream, shape, sigma, bf16=False, start=0):
    n = int(np.prod(shape))
    out = np.empty(n, np.float32)
    step = 1 << 22
    for a in range(0, n, step):
        c = min(step, n - a)
        out[a:a + c] = irwin_hall_np(seed, stream, start + a, c) * np.float32(sigma)
    if bf16:
        out = bf16_round_np(out)
    return out.reshape(shape)


def _to_i64(c):
    c &= _M64
    return c - (1 << 64) if c >= (1 << 63) else c


def normal_torch(seed, stream, shape, sigma, dtype, device, start=0):
    """Same values as normal_np, produced with torch integer ops on ``device``.

    ``dtype`` is torch.float32 or torch.bfloat16 (round-to-nearest-even cast).
    """
    import torch

    n = 1
    for d in shape:
        n *= int(d)
    out = torch.empty(n, dtype=dtype, device=device)
    base = _to_i64(stream_base(seed, stream))
    golden, c1, c2 = _to_i64(_GOLDEN), _to_i64(_C1), _to_i64(_C2)
    m34, m37, m33 = (1 << 34) - 1, (1 << 37) - 1, (1 << 33) - 1
    step = 1 << 24
    sig = torch.tensor(float(np.float32(sigma)), dtype=torch.float32, device=device)
    for a in range(0, n, step):
        c = min(step, n - a)
        i = torch.arange(start + a, start + a + c, dtype=torch.int64, device=device)
        s = torch.zeros(c, dtype=torch.int64, device=device)
        for j in range(3):
            z = (i * 3 + j) * golden + base
            z = (z ^ ((z >> 30) & m34)) * c1
            z = (z ^ ((z >> 27) & m37)) * c2
            z = z ^ ((z >> 31) & m33)
            for f in range(4):
                s += (z >> (16 * f)) & 0xFFFF
        v = (s - 6 * 65535).to(torch.float32) / 65536.0 * sig
        out[a:a + c] = v.to(dtype)
    return out.reshape(*shape)


def hot_experts(seed, E, count=4):
    """``count`` distinct expert ids chosen from the seed, ascending."""
    base = stream_base(seed, STREAM_HOT)
    chosen = []
    c = 0
    while len(chosen) < count:
        e = _mix64_int((base + c * _GOLDEN) & _M64) % E
        if e not in chosen:
            chosen.append(e)
        c += 1
    return sorted(chosen)


class MoeConfig:
    """One of the benchmark shapes."""

    def __init__(self, name, T, H, E, k, I, dtype, hot=0, hot_bias=3.0):
        self.name, self.T, self.H, self.E, self.k, self.I = name, T, H, E, k, I
        self.dtype, self.hot, self.hot_bias = dtype, hot, hot_bias

    def replace(self, **kw):
        c = MoeConfig(self.name, self.T, self.H, self.E, self.k, self.I, self.dtype,
                      self.hot, self.hot_bias)
        for a, b in kw.items():
            setattr(c, a, b)
        return c


CONFIGS = {
    "tiny_f32": MoeConfig("tiny_f32", 16, 256, 8, 2, 128, "f32"),
    "qwen3_30b_decode": MoeConfig("qwen3_30b_decode", 64, 2048, 128, 8, 768, "bf16"),
    "qwen3_30b_prefill": MoeConfig("qwen3_30b_prefill", 8192, 2048, 128, 8, 768, "bf16"),
    "qwen3_235b_t256": MoeConfig("qwen3_235b_t256", 256, 4096, 128, 8, 1536, "bf16"),
    "qwen3_235b_t4096": MoeConfig("qwen3_235b_t4096", 4096, 4096, 128, 8, 1536, "bf16"),
    "qwen3_30b_imbalance": MoeConfig("qwen3_30b_imbalance", 16384, 2048, 128, 8, 768,
                                     "bf16", hot=4),
}

SIGMA_W = 0.02
SIGMA_X = 1.0


def router_bias_np(cfg, seed):
    if not cfg.hot:
        return None
    b = np.zeros(cfg.E, np.float32)
    b[hot_experts(seed, cfg.E, cfg.hot)] = np.float32(cfg.hot_bias)
    return b


def make_inputs_np(cfg, seed=7907, tokens=None):
    """float32 numpy inputs (bf16-rounded values for bf16 configs).

    ``tokens`` optionally restricts the activations to a list of token ids.
    Returns dict(tokens, gate, ffn1, ffn2, bias).
    """
    bf = cfg.dtype == "bf16"
    gate = normal_np(seed, STREAM_GATE, (cfg.E, cfg.H), SIGMA_W, bf)
    ffn1 = normal_np(seed, STREAM_FFN1, (cfg.E, 2 * cfg.I, cfg.H), SIGMA_W, bf)
    ffn2 = normal_np(seed, STREAM_FFN2, (cfg.E, cfg.H, cfg.I), SIGMA_W, bf)
    if tokens is None:
        x = normal_np(seed, STREAM_TOKENS, (cfg.T, cfg.H), SIGMA_X, bf)
    else:
        x = np.stack([normal_np(seed, STREAM_TOKENS, (cfg.H,), SIGMA_X, bf, start=t * cfg.H)
                      for t in tokens])
    return dict(tokens=x, gate=gate, ffn1=ffn1, ffn2=ffn2, bias=router_bias_np(cfg, seed))


def make_inputs_torch(cfg, seed=7907, device="cuda"):
    """Device tensors in the layer's storage dtype. Same values as make_inputs_np."""
    import torch

    dt = torch.bfloat16 if cfg.dtype == "bf16" else torch.float32
    gate = normal_torch(seed, STREAM_GATE, (cfg.E, cfg.H), SIGMA_W, dt, device)
    ffn1 = normal_torch(seed, STREAM_FFN1, (cfg.E, 2 * cfg.I, cfg.H), SIGMA_W, dt, device)
    ffn2 = normal_torch(seed, STREAM_FFN2, (cfg.E, cfg.H, cfg.I), SIGMA_W, dt, device)
    x = normal_torch(seed, STREAM_TOKENS, (cfg.T, cfg.H), SIGMA_X, dt, device)
    b = router_bias_np(cfg, seed)
    bias = None if b is None else torch.from_numpy(b).to(device)
    return dict(tokens=x, gate=gate, ffn1=ffn1, ffn2=ffn2, bias=bias)
