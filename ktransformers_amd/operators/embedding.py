"""Injected token embeddings.  KSinusoidEmbedding: x[t] = table[token] + s(position), the fixed sinusoid
s(p)[2i] = sin(p base^(-2i / width)), s(p)[2i + 1] = cos(p base^(-2i / width)), written as the fp32 residual stream
(include/ktx_seq.h `ktx_embed_sinpos`: the angle and its sine in fp64, one rounding).  `base` is a constructor argument."""
from __future__ import annotations

import torch

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KSinusoidEmbedding(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 base: float = 10000.0, **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "base", float(base))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        dev = torch.device(self.device)
        table = self.gguf_loader.load_tensor(self.key, device=dev).to(self.compute_dtype).contiguous()
        width = table.shape[1]
        i = torch.arange((width + 1) // 2, dtype=torch.float64)
        self.w.update(table=table, inv_freq=torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / width).to(dev))

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        from ktransformers_amd._native_seq import embed_sinpos
        return embed_sinpos(tokens.reshape(-1).to(torch.int32), positions.reshape(-1).to(torch.int32), self.w["table"], self.w["inv_freq"])


class KTableEmbedding(BaseInjectedModule):
    """x[t] = table[token] written as the fp32 residual stream (positions enter elsewhere, e.g. by rotation in the attention);
    include/ktx_seq.h `ktx_embed_sinpos` without its positional term."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        self.w["table"] = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(self.compute_dtype).contiguous()

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        from ktransformers_amd._native_seq import embed_rows
        return embed_rows(tokens.reshape(-1).to(torch.int32), self.w["table"])


class KPassOffset(BaseInjectedModule):
    """What a block of layers that runs several times with the same weights adds to the residual stream in front of pass t:
    the embedding output again (every pass but the first) and a learned vector per pass, table[t] — one launch
    (include/ktx_hyb.h `ktx_rows_add`).  Checkpoint tensor: `<key>.step` [passes, width]."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 table_suffix: str = ".step", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "table_suffix", table_suffix)
        object.__setattr__(self, "w", {})

    def load(self):
        t = self.gguf_loader.load_tensor(self.key + self.table_suffix, device=torch.device(self.device)).to(torch.float32).contiguous()
        if t.dim() != 2 or t.shape[0] < self.orig_module.times:
            raise ValueError(f"{self.key}{self.table_suffix}: expected [passes >= {self.orig_module.times}, width], got {tuple(t.shape)}")
        self.w["step"] = t

    def forward(self, x: torch.Tensor, x0: torch.Tensor, t: int) -> torch.Tensor:
        from ktransformers_amd._native_hyb import rows_add
        return rows_add(x, x0 if t > 0 else None, self.w["step"][t])


class KScaledEmbedding(BaseInjectedModule):
    """x[t] = table[token] * scale as the fp32 residual stream.  The table is kept in fp32 with the scale folded in (the product
    of a bf16 entry and the scale, rounded once — what multiplying after the lookup gives); `scale` is read from the replaced module."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "scale", float(orig_module.scale))
        object.__setattr__(self, "w", {})

    def load(self):
        t = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(torch.float32)
        self.w["table"] = (t * self.scale).contiguous()

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        from ktransformers_amd._native_seq import embed_rows
        return embed_rows(tokens.reshape(-1).to(torch.int32), self.w["table"], out=out)


class KTokenSideTable(BaseInjectedModule):
    """The table behind per-layer token inputs: one row per token id, `layers * dim` entries, layer i reads [i * dim, (i + 1) * dim).
    Checkpoint tensor: `<key>.embed`."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 table_suffix: str = ".embed", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "table_suffix", table_suffix)
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        t = self.gguf_loader.load_tensor(self.key + self.table_suffix, device=torch.device(self.device)).to(self.compute_dtype).contiguous()
        if t.shape[1] < self.orig_module.layers * self.orig_module.dim:
            raise ValueError(f"{self.key}{self.table_suffix}: {tuple(t.shape)} holds fewer than {self.orig_module.layers} x {self.orig_module.dim} entries per token")
        self.w["table"] = t

    def forward(self):
        return self.w["table"]


class KTokenSideInput(BaseInjectedModule):
    """A per-layer input looked up by token: y = W_proj (gelu_tanh(W_gate x) * e), e = the layer's slice of the token's row in the side
    table; the caller adds y / rms(y) * w to the residual (operators/layernorm.py: the `y_norm` of the launch that follows).  The
    gate's activation rides in its GEMM's epilogue; the product with e is one small launch (`ktx_rows_mul_lookup`).
    Checkpoint tensors: `<key>.gate` [dim, width], `<key>.proj` [width, dim], `<key>.norm` [width]."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        for name in ("dim", "width", "layer_idx", "eps"):
            object.__setattr__(self, name, getattr(orig_module, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        dev, cd = torch.device(self.device), self.compute_dtype
        get = lambda n: self.gguf_loader.load_tensor(f"{self.key}.{n}", device=dev)
        self.w.update(gate=get("gate").to(cd).contiguous(), proj=get("proj").to(cd).contiguous(),
                      norm=get("norm").to(torch.float32).contiguous())
        if tuple(self.w["gate"].shape) != (self.dim, self.width) or tuple(self.w["proj"].shape) != (self.width, self.dim) or \
                self.w["norm"].numel() != self.width:
            raise ValueError(f"{self.key}: tensors do not fit dim={self.dim} width={self.width}")

    @property
    def y_norm(self):
        return self.w["norm"], self.eps

    def forward(self, x: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        """x fp32 [T, width] (the residual after the layer's sublayers), tokens int32 [T] -> y fp32 [T, width], not yet normed."""
        from ktransformers_amd._native_seq import dense_gemm, dense_gemm_skinny
        from ktransformers_amd._native_swa import rows_mul_lookup
        g = dense_gemm_skinny(x, self.w["gate"], act="gelu_tanh")
        ge = rows_mul_lookup(g, table, self.layer_idx * self.dim, tokens, out_dtype=self.compute_dtype)
        return dense_gemm(ge, self.w["proj"])
