"""Runs one MoE configuration through the C ABI on the GPU and through the CPU
oracle, and compares them. Used by the gpu-marked parity tests."""
import numpy as np
import torch

from flash_distributed_moe_amd import _lib, synth
from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher
from oracle import oracle
from tests.helpers import max_rel_err

# Output tolerance (max|got-ref| / max|ref|): bf16 layers against the
# float32-accumulated oracle on the same bf16-rounded inputs; float32 layers
# differ from the oracle only by MFMA summation order.
TOL = {"bf16": 1e-2, "f32": 2e-5}


class GpuCase:
    def __init__(self, cfg, seed=7907, sched=_lib.SCHED_AUTO, max_tokens=None, inputs=None,
                 pack_weights=False, prepacked=False, norm_weight=None, norm_eps=1e-6, residual=False):
        self.cfg, self.seed = cfg, seed
        self.pack_weights, self.prepacked = pack_weights, prepacked
        self.norm_weight, self.norm_eps, self.residual = norm_weight, norm_eps, residual
        self.dev = torch.device("cuda:0")
        self.inp = inputs or synth.make_inputs_torch(cfg, seed, self.dev)
        self.launcher = MoeKernelLauncher()
        uid = self.launcher.getDistributedUniqueId(empty=True)
        self.launcher.create(self.inp["gate"], self.inp["ffn1"], self.inp["ffn2"],
                             max_tokens or cfg.T, uid, 0, 1, top_k=cfg.k,
                             router_bias=self.inp["bias"], sched=sched,
                             pack_weights=pack_weights, prepacked=prepacked,
                             norm_weight=norm_weight, norm_eps=norm_eps, residual=residual)

    def run(self, tokens=None, inplace=False):
        x = self.inp["tokens"] if tokens is None else tokens
        if inplace:
            buf = x.clone()
            self.launcher.launch(buf, buf)
            out = buf
        else:
            out = torch.full_like(x, float("nan"))
            self.launcher.launch(x, out)
        torch.cuda.synchronize()
        err, _ = self.launcher.status()
        assert err == 0, "device error bits %d" % err
        return out

    def close(self):
        self.launcher.destroy()

    # ------------------------------------------------------------- oracle side
    def host_weights(self):
        if not hasattr(self, "_hw"):
            self._hw = {k: (None if self.inp[k] is None else self.inp[k].float().cpu().numpy())
                        for k in ("gate", "ffn1", "ffn2", "bias")}
        return self._hw

    def layer_input(self, x):
        """What the router and the experts see: the rows, or their RMSNorm."""
        if self.norm_weight is None:
            return x
        return oracle.rmsnorm(x, self.norm_weight.float().cpu().numpy(), self.norm_eps,
                              bf16=self.cfg.dtype == "bf16")

    def check_routing(self, tokens_t, routing):
        """Bit-exact top-k indices, counts, offsets and permutation; weights to 1e-6."""
        hw = self.host_weights()
        x = self.layer_input(tokens_t.float().cpu().numpy())
        idx, w = oracle.gate(x, hw["gate"], self.cfg.k, bias=hw["bias"])
        assert np.array_equal(routing["topk_idx"], idx), "top-k indices differ from the oracle"
        np.testing.assert_allclose(routing["topk_w"], w, rtol=2e-6, atol=1e-7)
        counts, offsets, perm = oracle.permute(idx, self.cfg.E)
        assert np.array_equal(routing["counts"], counts)
        assert np.array_equal(routing["offsets"], offsets)
        assert np.array_equal(routing["perm"], perm), "per-expert permutation differs"
        return idx, w

    def check_outputs(self, tokens_t, out_t, token_ids=None, nthreads=1):
        """Outputs of the chosen tokens (all when None) against the oracle."""
        hw = self.host_weights()
        x = tokens_t.float().cpu().numpy()
        got = out_t.float().cpu().numpy()
        if token_ids is not None:
            x, got = x[token_ids], got[token_ids]
        gamma = None if self.norm_weight is None else self.norm_weight.float().cpu().numpy()
        ref, _, _ = oracle.layer(x, hw["gate"], hw["ffn1"], hw["ffn2"], self.cfg.k, bias=hw["bias"],
                                 norm_weight=gamma, norm_eps=self.norm_eps, residual=self.residual,
                                 bf16=self.cfg.dtype == "bf16", nthreads=nthreads)
        assert np.all(np.isfinite(got)), "non-finite output"
        err = max_rel_err(got, ref)
        tol = TOL[self.cfg.dtype]
        assert err <= tol, "max relative error %.3e > %.1e" % (err, tol)
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        # elementwise as well: bf16 layers round every expert contribution of the tiled variant
        # to bf16 before the slot sum, whose tail over 10^7 elements reaches 1.5 * tol * rms
        np.testing.assert_allclose(got, ref, rtol=tol, atol=tol * rms * (2 if self.cfg.dtype == "bf16" else 1))
        return err
