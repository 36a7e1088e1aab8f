"""Causal convolution over time on what a sublayer reads — an injected operator for decoders on an fp32 residual stream:

    h_t <- h_t + sum_j w[:, j] * h_(t - taps + 1 + j)        (per channel; zeros before the sequence's start; no bias)

The operator only holds the taps (fp32 [width, taps]; the last column multiplies the current token); the arithmetic is the second
launch of the norm in front of it (operators/layernorm.py KScalarRMSNorm -> include/ktx_swa.h `ktx_resid_norm`, `ktx_input_conv`).
The last taps - 1 inputs of every sequence are state: the cache manager keeps them per request slot (KHybridCache spec "pre").
Checkpoint tensor: the module's key."""
from __future__ import annotations

import torch

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KInputConv(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "taps", int(orig_module.taps))
        object.__setattr__(self, "width", int(orig_module.width))
        object.__setattr__(self, "weight_f32", None)

    def load(self):
        w = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(torch.float32).contiguous()
        if tuple(w.shape) != (self.width, self.taps):
            raise ValueError(f"{self.key}: expected [{self.width}, {self.taps}], got {tuple(w.shape)}")
        object.__setattr__(self, "weight_f32", w)

    def forward(self, *args, **kwargs):
        raise RuntimeError(f"{self.key}: the input convolution runs inside the norm in front of it (KScalarRMSNorm.forward(conv=...))")
