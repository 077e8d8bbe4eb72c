"""Python surface of the launcher, mirroring the reference's ``flashMoeLauncher``
extension (python/pyMoeLauncherTorch.cpp:115-133): class ``MoeKernelLauncher``
with ``getDistributedUniqueId / create / launch / destroy / valid``.

Same argument meaning, checks and error behaviour as the reference binding
(tensor checks pyMoeLauncherTorch.cpp:24-31, shape relations :81-87, uid length
:100-101, "Launcher was destroyed" :45, current torch stream :58,65,93), with
these additions: bfloat16 tensors are accepted next to float32, and ``create``
takes optional ``top_k`` (default 8, the reference's compile-time value),
``router_bias``, ``sched`` and ``pack_weights`` (keep a streaming-friendly second
copy of the expert weights for small batches). torch supplies device memory and the current
stream; the work happens behind the C ABI of libflashMoe.so.
"""
import ctypes

import numpy as np
import torch

from . import _lib

_UID_BYTES = 128


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _check_tensor(t, name, dtypes=(torch.float32, torch.bfloat16)):
    _check(isinstance(t, torch.Tensor), "%s tensor is undefined" % name)
    _check(t.is_cuda, "%s must be a CUDA tensor (ROCm)" % name)
    _check(t.dtype in dtypes, "%s must be float32 or bfloat16" % name)
    _check(t.is_contiguous(), "%s must be contiguous" % name)


def _hip_check(code, what):
    if code != _lib.HIP_SUCCESS:
        raise RuntimeError("%s failed with hipError_t %d" % (what, code))


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class MoeKernelLauncher:
    def __init__(self):
        self._h = None
        self._lib = _lib.load()
        self._dtype = None
        self._shape = None
        self._keep = None

    @staticmethod
    def getDistributedUniqueId(empty=False):
        """128 zero bytes: there is no inter-GPU transport to identify."""
        return bytes(_UID_BYTES)

    @property
    def valid(self):
        return self._h is not None

    def create(self, gate_weights, ffn1_expert_weights, ffn2_expert_weights, max_tokens, uid,
               rank, world_size, top_k=8, router_bias=None, sched=_lib.SCHED_AUTO,
               pack_weights=None, prepacked=False, norm_weight=None, norm_eps=1e-6, residual=False):
        """pack_weights left out (as in a call written against the reference): the launcher keeps
        a packed copy of the expert weights, unless they are prepacked; False reads the row-major
        tensors. norm_weight ([H], the weights' dtype): the layer runs on rmsnorm(tokens) with
        this weight and norm_eps; residual: the input rows are added to the output."""
        if pack_weights is None:
            pack_weights = not prepacked
        _check(self._h is None, "Launcher already created")
        for t, n in ((gate_weights, "gate_weights"), (ffn1_expert_weights, "ffn1_expert_weights"),
                     (ffn2_expert_weights, "ffn2_expert_weights")):
            _check(isinstance(t, torch.Tensor), "%s tensor is undefined" % n)
        _check(gate_weights.dim() == 2 and ffn1_expert_weights.dim() == 3
               and ffn2_expert_weights.dim() == 3, "weights must be [E,H], [E,2I,H], [E,H,I]")
        experts, hidden = gate_weights.shape
        inter = ffn2_expert_weights.shape[2]
        _check(world_size > 0, "world_size must be positive")
        _check(ffn1_expert_weights.shape[0] == experts // world_size, "ffn1 expert count")
        _check(ffn1_expert_weights.shape[1] == 2 * inter, "ffn1 rows must be 2*intermediate")
        _check(ffn1_expert_weights.shape[2] == hidden, "ffn1 hidden size")
        _check(ffn2_expert_weights.shape[0] == experts // world_size, "ffn2 expert count")
        _check(ffn2_expert_weights.shape[1] == hidden, "ffn2 hidden size")
        _check_tensor(gate_weights, "gate_weights")
        _check_tensor(ffn1_expert_weights, "ffn1_expert_weights")
        _check_tensor(ffn2_expert_weights, "ffn2_expert_weights")
        _check(gate_weights.dtype == ffn1_expert_weights.dtype == ffn2_expert_weights.dtype,
               "all weights must share one dtype")
        _check(isinstance(uid, (bytes, bytearray)) and len(uid) == _UID_BYTES,
               "uid must be 128 bytes")
        _check(world_size == 1 and rank == 0,
               "only rank 0 of a world of 1 is supported (no inter-GPU transport)")
        if router_bias is not None:
            _check_tensor(router_bias, "router_bias", (torch.float32,))
            _check(tuple(router_bias.shape) == (experts,), "router_bias must be [E]")

        d = _lib.LayerDesc()
        d.experts, d.hidden, d.intermediate, d.top_k = experts, hidden, inter, int(top_k)
        d.dtype = _lib.BF16 if gate_weights.dtype == torch.bfloat16 else _lib.F32
        d.max_tokens, d.sched = int(max_tokens), int(sched)
        _check(not (pack_weights and prepacked), "prepacked weights need no packed copy")
        d.flags = (_lib.FLAG_PACK_WEIGHTS if pack_weights else 0) | \
                  (_lib.FLAG_WEIGHTS_PREPACKED if prepacked else 0)
        d.gate_weights = gate_weights.data_ptr()
        d.ffn1_weights = ffn1_expert_weights.data_ptr()
        d.ffn2_weights = ffn2_expert_weights.data_ptr()
        d.router_bias = router_bias.data_ptr() if router_bias is not None else None
        if norm_weight is not None:
            _check_tensor(norm_weight, "norm_weight", (gate_weights.dtype,))
            _check(tuple(norm_weight.shape) == (hidden,), "norm_weight must be [H]")
            d.flags |= _lib.FLAG_RMSNORM
            d.norm_weight, d.norm_eps = norm_weight.data_ptr(), float(norm_eps)
        if residual:
            d.flags |= _lib.FLAG_RESIDUAL
        h = ctypes.c_void_p()
        with torch.cuda.device(gate_weights.device):
            _hip_check(self._lib.flashMoeCreate(ctypes.byref(h), ctypes.byref(d), _stream()),
                       "CreateLauncher")
        self._h = h
        self._dtype = gate_weights.dtype
        self._shape = (experts, hidden, inter, int(top_k))
        # weights are borrowed by the library: keep them alive with the launcher
        self._keep = (gate_weights, ffn1_expert_weights, ffn2_expert_weights, router_bias, norm_weight)
        self._device = gate_weights.device

    @staticmethod
    def pack_weights_in_place(ffn1_expert_weights, ffn2_expert_weights):
        """Rewrites the two expert tensors ([E,2I,H], [E,H,I]) into the packed layout where
        they lie (no second copy); pass them to create(..., prepacked=True) afterwards.
        Their contents are no longer row-major matrices after this."""
        lib = _lib.load()
        _check_tensor(ffn1_expert_weights, "ffn1_expert_weights")
        _check_tensor(ffn2_expert_weights, "ffn2_expert_weights")
        experts, two_i, hidden = ffn1_expert_weights.shape
        inter = two_i // 2
        _check(tuple(ffn2_expert_weights.shape) == (experts, hidden, inter), "ffn2 must be [E,H,I]")
        dt = _lib.BF16 if ffn1_expert_weights.dtype == torch.bfloat16 else _lib.F32
        with torch.cuda.device(ffn1_expert_weights.device):
            for which, t in ((0, ffn1_expert_weights), (1, ffn2_expert_weights)):
                _hip_check(lib.flashMoePackWeightsInPlace(dt, experts, hidden, inter, which,
                                                          t.data_ptr(), _stream()),
                           "flashMoePackWeightsInPlace")

    def launch(self, tokens, output):
        if self._h is None:
            raise RuntimeError("Launcher was destroyed")
        _check_tensor(tokens, "tokens", (self._dtype,))
        _check_tensor(output, "output", (self._dtype,))
        _check(tokens.dim() == 2 and tokens.shape[1] == self._shape[1],
               "tokens must be [tokens, hidden]")
        _check(tuple(output.shape) == tuple(tokens.shape), "output shape must equal tokens shape")
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeLaunch(self._h, tokens.data_ptr(), output.data_ptr(),
                                                int(tokens.shape[0]), _stream()), "Launch")

    def destroy(self):
        if self._h is not None:
            with torch.cuda.device(self._device):
                _hip_check(self._lib.flashMoeDestroy(self._h, _stream()), "DestroyLauncher")
            self._h = None
            self._keep = None

    # ---- additions for tests and diagnostics (no counterpart in the reference)
    def routing(self, tokens_num):
        """Routing of the last launch: dict of numpy arrays."""
        if self._h is None:
            raise RuntimeError("Launcher was destroyed")
        E, _, _, k = self._shape
        idx = np.empty((tokens_num, k), np.int32)
        w = np.empty((tokens_num, k), np.float32)
        counts = np.empty(E, np.int32)
        offsets = np.empty(E + 1, np.int32)
        perm = np.empty(tokens_num * k, np.int32)
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeReadRouting(
                self._h, tokens_num, idx.ctypes.data, w.ctypes.data, counts.ctypes.data,
                offsets.ctypes.data, perm.ctypes.data, _stream()), "flashMoeReadRouting")
        return dict(topk_idx=idx, topk_w=w, counts=counts, offsets=offsets,
                    perm=perm[:int(offsets[E])])

    def intermediate(self, tokens_num):
        """h of the last launch as float32 [tokens_num*k, I], rows in permuted order."""
        if self._h is None:
            raise RuntimeError("Launcher was destroyed")
        _, _, inter, k = self._shape
        raw = np.empty((tokens_num * k, inter), np.uint16 if self._dtype == torch.bfloat16 else np.float32)
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeReadIntermediate(self._h, tokens_num, raw.ctypes.data, _stream()),
                       "flashMoeReadIntermediate")
        if raw.dtype == np.uint16:
            return (raw.astype(np.uint32) << 16).view(np.float32)
        return raw

    def down_rows(self, tokens_num):
        """(y, weighted): the down projection's rows of the last launch as float32
        [tokens_num*k, H], row t*k+slot, and whether they already carry the slot's gate
        weight (the streaming variant's do, the tiled variant's do not)."""
        if self._h is None:
            raise RuntimeError("Launcher was destroyed")
        _, hidden, _, k = self._shape
        raw = np.empty((tokens_num * k, hidden), np.float32)
        dtype, weighted = ctypes.c_int(-1), ctypes.c_int(-1)
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeReadDownRows(self._h, tokens_num, raw.ctypes.data, ctypes.byref(dtype),
                                                      ctypes.byref(weighted), _stream()), "flashMoeReadDownRows")
        if dtype.value == _lib.BF16:
            bits = raw.view(np.uint16).reshape(-1)[:tokens_num * k * hidden]
            raw = (bits.astype(np.uint32) << 16).view(np.float32).reshape(tokens_num * k, hidden)
        return raw, bool(weighted.value)

    def status(self):
        """(error_bits, completed_launches) after waiting for the current stream."""
        err, n = ctypes.c_uint(), ctypes.c_uint()
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeStatus(self._h, ctypes.byref(err), ctypes.byref(n),
                                                _stream()), "flashMoeStatus")
        return err.value, n.value

    def set_wait_limit_ms(self, ms):
        _hip_check(self._lib.flashMoeSetWaitLimitMs(self._h, float(ms)), "flashMoeSetWaitLimitMs")

    TRACE_DTYPE = np.dtype([("ticket", "<u4"), ("kind", "<u4"), ("worker", "<u4"), ("aux", "<u4"),
                            ("t_fetch", "<i8"), ("t_ready", "<i8"), ("t_end", "<i8"),
                            ("x0", "<u4"), ("x1", "<u4")])  # spare words (timing experiments)

    def trace_enable(self, capacity):
        _hip_check(self._lib.flashMoeTraceEnable(self._h, int(capacity)), "flashMoeTraceEnable")
        self._trace_cap = int(capacity)

    def trace_read(self):
        """Records of the traced launches since the last read (numpy structured array)."""
        rec = np.empty(self._trace_cap, self.TRACE_DTYPE)
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeTraceRead(self._h, rec.ctypes.data, self._trace_cap,
                                                   _stream()), "flashMoeTraceRead")
        return rec[rec["kind"] != 0xFFFFFFFF]

    def refresh_weights(self):
        """Re-pack the expert weights after the caller changed them in place."""
        with torch.cuda.device(self._device):
            _hip_check(self._lib.flashMoeRefreshWeights(self._h, _stream()),
                       "flashMoeRefreshWeights")

    def sched_for(self, tokens_num):
        return self._lib.flashMoeSchedFor(self._h, int(tokens_num))
