"""Grouped-query sliding-window attention with rotated values and a sink — an injected operator beside the MLA and latent-window
operators (operators/attention.py, latent_window_attention.py) for decoders on an fp32 residual stream, any sizes, bf16 or fp32:

    q = W_q h [heads, dim], k = W_k h [kv_heads, dim], v = W_v h [kv_heads, vdim]; query head h reads key head h // (heads / kv_heads);
    the first rot_dims entries of every q and k head turn with the position p (pairs (2i, 2i + 1), angle p base^(-2i / rot_dims));
    then q and k are divided by their RMS over dim (no weight);
    the value of position j is turned by j over ALL its entries (pairs (2m, 2m + 1), angle j base^(-2m / vdim)) and cached so; a
    head's weighted sum at position i is turned back by i — values enter relative to the query;
    score = scale (q . k); position i sees j with 0 <= i - j < window;
    weights p_j = exp(s_j) / (e^sink + sum_j exp(s_j)): a sink that takes weight and gives no value (with score 0 the extra term is 1);
    W_o on the concatenated heads.

Rotated, normed keys and rotated values are appended to the KHybridCache's paged key / value caches (spec "kv") by the prep launch;
prompts, portions and decode steps are one pass over them (include/ktx_swa.h `ktx_swa_prep`, `ktx_swa_mfma` on the matrix cores for
bf16 caches, `ktx_swa_forward` on the vector ALUs for fp32 and odd sizes).  Angles, scores and softmax are fp32.  window, scale, the
rotation's base and span, the sink's score, eps and the q / k norm are constructor arguments (read from the replaced module).

Further options, each off unless the replaced module names it:
    qkv_bias / out_bias   the projections have biases (`<key>.q.b` ..; the output's is handed to the caller as `out_bias`: it joins the
                          residual in the norm's launch);
    conv_taps             a causal convolution over time on every channel of q, k and v directly behind the projections
                          (`<key>.q.conv` .. [channels, taps]); the last taps - 1 projected rows of a sequence are state (spec "conv");
    proj_norm             q and k are RMS-normed over their WHOLE projection (all heads at once) with weights `<key>.q.norm`, `<key>.k.norm`;
    dist_far              a learned bias by distance is added to the scaled score, `<key>.rel` [rows, heads]: distances below rows / 2
                          have a row each, the rest share rows on a logarithmic scale that reaches the last row at distance dist_far;
    keep_first            the sequence's first positions stay visible behind the window;
    sink = "learned"      the sink's score is `<key>.sink` [heads].
With any of the first three the prep is `ktx_swa_conv_prep` (no rotation in that form)."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KWindowGQAttention(BaseInjectedModule):
    TARGET_WORKGROUPS = 1024
    KEYS_PER_SPLIT = 64
    USE_MATRIX_CORES = True

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("heads", "kv_heads", "dim", "vdim", "rot_dims", "rot_base", "rot_values", "qk_norm", "sink_score", "scale", "window",
                     "eps", "width"):
            object.__setattr__(self, name, getattr(o, name))
        for name, default in (("qkv_bias", False), ("out_bias_on", False), ("conv_taps", 0), ("proj_norm", False), ("dist_far", None),
                              ("keep_first", 0), ("sink", None)):
            object.__setattr__(self, name, getattr(o, name, default))
        object.__setattr__(self, "conv_form", bool(self.qkv_bias or self.conv_taps or self.proj_norm))
        if self.conv_form and (self.rot_dims or self.rot_values or self.qk_norm):
            raise ValueError(f"{key}: biases, a convolution or whole-projection norms go with un-rotated, un-normed heads")
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_cfg", {})

    def state_spec(self) -> dict:
        spec = {"kv": (self.kv_heads, self.dim, self.vdim)}
        if self.conv_taps > 1:
            spec["conv"] = (self.heads * self.dim + self.kv_heads * (self.dim + self.vdim), self.conv_taps)
        return spec

    @property
    def out_bias(self):
        return self.w.get("o_b")

    @staticmethod
    def distance_rows(rows: int, far: float) -> list:
        """Row of a [rows, heads] distance table for each distance 0 .. ceil(far): the first rows / 2 distances have a row each, the rest
        share rows on a logarithmic scale that reaches the last row at distance `far` (every larger distance reads the last row)."""
        import math
        half = rows // 2
        out = []
        for n in range(int(math.ceil(far)) + 1):
            out.append(n if n < half else min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
        return out

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        H, G, D, V = self.heads, self.kv_heads, self.dim, self.vdim
        get = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(cd)
        q, k, v, o = get("q"), get("k"), get("v"), get("o")
        if tuple(q.shape) != (H * D, self.width) or tuple(k.shape) != (G * D, self.width) or tuple(v.shape) != (G * V, self.width) or \
                tuple(o.shape) != (self.width, H * V):
            raise ValueError(f"{self.key}: tensor shapes do not fit heads={H} kv_heads={G} dim={D} vdim={V} width={self.width}")
        self.w.update(qkv=torch.cat([q, k, v]).contiguous(), o=o.contiguous())
        f64 = lambda n: torch.pow(torch.tensor(float(self.rot_base), dtype=torch.float64),
                                  -2.0 * torch.arange(n // 2, dtype=torch.float64) / max(n, 1)).to(dev)
        self.w["inv_freq"] = f64(self.rot_dims) if self.rot_dims else None
        self.w["v_inv_freq"] = f64(V) if self.rot_values else None
        self.w["sink"] = None if self.sink_score is None else torch.full((H,), float(self.sink_score), dtype=torch.float32, device=dev)
        f32 = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(torch.float32).contiguous()
        if self.sink == "learned":
            self.w["sink"] = f32("sink").reshape(-1)
            if self.w["sink"].numel() != H:
                raise ValueError(f"{self.key}.sink: one score per head")
        if self.qkv_bias:
            self.w["qkv_b"] = torch.cat([f32("q.b"), f32("k.b"), f32("v.b")]).contiguous()
        if self.out_bias_on:
            self.w["o_b"] = f32("o.b")
        if self.conv_taps:
            self.w["conv"] = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")]).contiguous()
            if tuple(self.w["conv"].shape) != ((H + G) * D + G * V, self.conv_taps):
                raise ValueError(f"{self.key}: convolution weights must be [channels, {self.conv_taps}]")
        if self.proj_norm:
            self.w["q_norm"], self.w["k_norm"] = f32("q.norm").reshape(-1), f32("k.norm").reshape(-1)
        self.w["dist_bias"] = None
        if self.dist_far is not None:
            rel, far = f32("rel"), float(self.dist_far)
            rows = rel.shape[0]
            if rel.dim() != 2 or rel.shape[1] != H or rows < 2 or far <= rows // 2:
                raise ValueError(f"{self.key}.rel: expected [rows >= 2, {H}] and a far distance beyond rows / 2")
            # the table by DISTANCE: the kernels index it with min(i - j, its last row)
            self.w["dist_bias"] = rel[torch.tensor(self.distance_rows(rows, far), device=dev)].contiguous()

    def _config(self, cache):
        from ktransformers_amd._native_swa import swa_config
        k = (cache.page_size, cache.dtype)
        if k not in self._cfg:
            self._cfg[k] = swa_config(self.heads, self.kv_heads, self.dim, self.vdim, self.rot_dims, self.rot_values, self.qk_norm,
                                      self.eps, self.scale, self.window or 0, cache.page_size, cache.dtype, keep_first=self.keep_first,
                                      bias_span=0 if self.w["dist_bias"] is None else self.w["dist_bias"].shape[0] - 1)
        return self._cfg[k]

    def forward(self, h: torch.Tensor, batch, cache, cache_idx: int) -> torch.Tensor:
        """h [T, width] in the compute type -> W_o(attention) fp32 [T, width]; the step's key and value rows are appended to the cache."""
        from ktransformers_amd._native_seq import dense_gemm
        from ktransformers_amd._native_swa import swa_conv_prep, swa_forward, swa_mfma, swa_mfma_eligible, swa_prep
        H, G, D = self.heads, self.kv_heads, self.dim
        cfg, T = self._config(cache), h.shape[0]
        kc, vc = cache.k_caches[cache_idx], cache.v_caches[cache_idx]
        proj = dense_gemm(h, self.w["qkv"])
        if self.conv_form:
            q, vcs = swa_conv_prep(cfg, proj, self.w.get("qkv_b"), self.w.get("conv"), self.w.get("q_norm"), self.w.get("k_norm"), batch,
                                   cache.conv[cache_idx] if self.conv_taps > 1 else None, kc, vc), None
        else:
            q, vcs = swa_prep(cfg, proj, 0, H * D, (H + G) * D, self.w["inv_freq"], self.w["v_inv_freq"], batch.positions, batch.cache_loc, kc, vc)
        bias = self.w["dist_bias"]
        span = batch.max_kv_len if not self.window else min(batch.max_kv_len, self.window + self.keep_first + batch.max_q_len)
        if self.USE_MATRIX_CORES and kc.dtype == torch.bfloat16 and swa_mfma_eligible(cfg):
            blocks = batch.B * G * ((batch.max_q_len * (H // G) + 63) // 64)
            nsplit = max(1, min(self.TARGET_WORKGROUPS // max(blocks, 1), (span + self.KEYS_PER_SPLIT - 1) // self.KEYS_PER_SPLIT))
            o = swa_mfma(cfg, q, kc, vc, batch, self.w["sink"], vcs, nsplit=nsplit, out_dtype=self.compute_dtype, dist_bias=bias)
        else:
            span = batch.max_kv_len if not self.window else min(batch.max_kv_len, self.window + self.keep_first)
            nsplit = max(1, min(self.TARGET_WORKGROUPS // max(T * G, 1), (span + self.KEYS_PER_SPLIT - 1) // self.KEYS_PER_SPLIT))
            o = swa_forward(cfg, q, kc, vc, batch, self.w["sink"], vcs, nsplit=nsplit, out_dtype=self.compute_dtype, dist_bias=bias)
        return dense_gemm(o, self.w["o"])
