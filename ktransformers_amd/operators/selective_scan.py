"""Selective-scan mixer (Mamba) — an injected recurrent operator beside operators/mlstm.py and delta_rule.py for decoders on an fp32
residual stream, any sizes, bf16 or fp32:

    W_in h = [x | z] (inner channels each);  x <- silu(conv(x) + b) with a causal convolution per channel;
    W_x x = [dt_low (dt_rank) | B (state) | C (state)];  dt = softplus(W_dt dt_low + dt_bias), one per channel;  A = -exp(A_log);
    per channel c and state entry n:  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c;
    out = W_o (y * silu(z)).

S (fp32 [inner, state] per sequence) and the convolution's last taps - 1 inputs live in the KHybridCache's slots (specs "ssm", "conv")
and are carried from step to step; a sequence that starts at position 0 starts from zero.  Steps, decays, exponentials and the state are
fp32 (include/ktx_swa.h `ktx_ssm_conv`, `ktx_ssm_scan`).  Checkpoint tensors: `<key>.in`, `.conv`, `.conv.b`, `.x`, `.dt`, `.dt.b`,
`.A_log`, `.D`, `.o`."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KSelectiveScanMixer(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        for name in ("inner", "state", "dt_rank", "taps", "width"):
            object.__setattr__(self, name, getattr(orig_module, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_cfg", None)

    def state_spec(self) -> dict:
        return {"ssm": (self.inner, self.state), "conv": (self.inner, self.taps)}

    def load(self):
        from ktransformers_amd._native_swa import ssm_config
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        I, N, R = self.inner, self.state, self.dt_rank
        get = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev)
        f32 = lambda n: get(n).to(torch.float32).contiguous()
        self.w.update({"in": get("in").to(cd).contiguous(), "x": get("x").to(cd).contiguous(), "dt": get("dt").to(cd).contiguous(),
                       "o": get("o").to(cd).contiguous(), "conv": f32("conv"), "dt_b": f32("dt.b"), "A_log": f32("A_log"), "D": f32("D"),
                       "conv_b": f32("conv.b") if ld.has_tensor(f"{self.key}.conv.b") else None})
        if tuple(self.w["in"].shape) != (2 * I, self.width) or tuple(self.w["x"].shape) != (R + 2 * N, I) or \
                tuple(self.w["dt"].shape) != (I, R) or tuple(self.w["o"].shape) != (self.width, I) or \
                tuple(self.w["conv"].shape) != (I, self.taps) or tuple(self.w["A_log"].shape) != (I, N):
            raise ValueError(f"{self.key}: tensor shapes do not fit inner={I} state={N} dt_rank={R} taps={self.taps} width={self.width}")
        object.__setattr__(self, "_cfg", ssm_config(I, N, R, self.taps))

    def forward(self, h: torch.Tensor, batch, cache, cache_idx: int) -> torch.Tensor:
        """h [T, width] in the compute type -> W_o(gated scan output) fp32 [T, width]; the slots' state moves on."""
        from ktransformers_amd._native_seq import dense_gemm, dense_gemm_skinny
        from ktransformers_amd._native_swa import ssm_conv, ssm_scan
        I, N, R = self.inner, self.state, self.dt_rank
        S, cs = cache.S[cache_idx], cache.conv[cache_idx]
        proj = dense_gemm(h, self.w["in"])                                   # [x | z], fp32
        xc = ssm_conv(self._cfg, proj, 0, self.w["conv"], self.w["conv_b"], batch, cs)
        low = dense_gemm_skinny(xc, self.w["x"])                                   # [dt_low | B | C], fp32
        dt_raw = dense_gemm(low[:, :R], self.w["dt"])
        y = ssm_scan(self._cfg, xc, low[:, R:R + N], low[:, R + N:], dt_raw, self.w["dt_b"], self.w["A_log"], self.w["D"], proj, 0, I, batch,
                     S, cs, out_dtype=self.compute_dtype)
        return dense_gemm(y, self.w["o"])
