"""Sliding-window latent attention with a softmax sink — an injected operator beside the MLA ones (operators/attention.py) for decoders
on an fp32 residual stream, any sizes, bf16 or fp32:

    q = W_q h, per head [dim un-rotated | rot_dim rotated];  W_dkv h = [kv_rank | rot_dim]: the first part RMS-normed (weight
    `<key>.dkv.norm`) is the latent c, the second one rotated key part shared by the heads; per head k = [W_uk c | rotated part],
    v = W_uv c;  rotation of the first rot_dims entries of the rotated parts, pairs (2i, 2i + 1), angle p base^(-2i / rot_dims);
    position i sees j with 0 <= i - j < window;  softmax over the scores (times scale) AND one learned sink per head that has no value;
    W_o on the concatenated heads.

Only c and the rotated key part are cached (one row of kv_rank + rot_dim per token in the KHybridCache's paged latent cache).  The
products with W_uk and W_uv are moved to the query and the output side (q_lat = W_uk^T q, out = W_uv sum_j w_j c_j), so attention is
one pass over latent rows whatever the step brings: a prompt, a portion of one, or decode steps (include/ktx_hyb.h `ktx_latattn_prep`,
`ktx_grouped_gemm`, `ktx_latattn_forward`).  Scores, softmax, the sink and the rotation are fp32.  window, scale, the rotation's base and
span and eps are constructor arguments (read from the replaced module).

Options, each off unless the replaced module names it: `has_sink` = False: an ordinary softmax (no `<key>.sink`); `rot_half`: the
turning pairs are (i, i + rot_dims / 2) instead of neighbours; `gated`: the concatenated heads are multiplied by sigmoid(W_g h)
(`<key>.g` [heads * vdim, width], one more block of the input product) before W_o; `kv_from` = j: the layer has no down projection and
reads the latent rows that the layer with cache index j appended in the same step (equal kv_rank, rot_dim and rotation), with its own
W_uk, W_uv, queries and window."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule
from ktransformers_amd.operators.linear import merged_input_weight


class KLatentWindowAttention(BaseInjectedModule):
    TARGET_WORKGROUPS = 1024
    KEYS_PER_SPLIT = 64
    MFMA_KEYS_PER_SPLIT = 64
    USE_MATRIX_CORES = True

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot_dims", "rot_base", "scale", "window", "eps", "width"):
            object.__setattr__(self, name, getattr(o, name))
        for name, default in (("has_sink", True), ("rot_half", False), ("gated", False), ("kv_from", None)):
            object.__setattr__(self, name, getattr(o, name, default))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_cfg", {})
        object.__setattr__(self, "_merged", {})

    def state_spec(self) -> dict:
        return {} if self.kv_from is not None else {"latent": self.kv_rank + self.rot_dim}

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        H, D, R, V, L = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        get = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev)
        own = self.kv_from is None
        self.w.update(q=get("q").to(cd).contiguous(), dkv=get("dkv").to(cd).contiguous() if own else None, o=get("o").to(cd).contiguous(),
                      # per head W_uk^T [L, D] (the query side takes it) and W_uv [V, L]
                      ukT=get("uk").to(cd).reshape(H, D, L).transpose(1, 2).contiguous(),
                      uv=get("uv").to(cd).reshape(H, V, L).contiguous(),
                      lat_norm=get("dkv.norm").to(torch.float32).contiguous() if own else None,
                      sink=get("sink").to(torch.float32).contiguous() if self.has_sink else None,
                      g=get("g").to(cd).contiguous() if self.gated else None)
        if tuple(self.w["q"].shape) != (H * (D + R), self.width) or (own and tuple(self.w["dkv"].shape) != (L + R, self.width)) or \
                tuple(self.w["o"].shape) != (self.width, H * V) or (self.has_sink and self.w["sink"].numel() != H) or \
                (self.gated and tuple(self.w["g"].shape) != (H * V, self.width)):
            raise ValueError(f"{self.key}: tensor shapes do not fit heads={H} dim={D} rot_dim={R} vdim={V} kv_rank={L} width={self.width}")
        i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
        self.w["inv_freq"] = torch.pow(torch.tensor(float(self.rot_base), dtype=torch.float64), -2.0 * i / max(self.rot_dims, 1)).to(dev)

    def _config(self, cache):
        from ktransformers_amd._native_hyb import latattn_config
        k = (cache.page_size, cache.dtype)
        if k not in self._cfg:
            self._cfg[k] = latattn_config(self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank, self.rot_dims, self.scale,
                                          self.window or 0, self.eps, cache.page_size, cache.dtype, rot_half=self.rot_half)
        return self._cfg[k]

    def _input_weight(self, rider):
        k = id(rider) if rider is not None else None
        if k not in self._merged:
            self._merged[k] = merged_input_weight([t for t in (self.w["q"], self.w["dkv"], self.w["g"]) if t is not None], rider)
        return self._merged[k]

    def forward(self, h: torch.Tensor, batch, cache, cache_idx: int, rider=None):
        """h [T, width] in the compute type.  Returns (W_o(attention) fp32 [T, width], the rider's product or None); the step's latent
        rows are appended to the cache."""
        from ktransformers_amd._native_hyb import head_gemm, latattn_forward, latattn_mfma, latattn_mfma_eligible, latattn_prep
        from ktransformers_amd._native_seq import dense_gemm
        H, D, R, V, L = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        cfg, T = self._config(cache), h.shape[0]
        proj = dense_gemm(h, self._input_weight(rider))
        from ktransformers_amd._native_hyb import sigmoid_gate_rows
        own = self.kv_from is None
        c_off = H * (D + R)
        g_off = c_off + (L + R if own else 0)
        lat = cache.lat_caches[cache_idx if own else self.kv_from]
        if lat is None:
            raise ValueError(f"{self.key}: cache entry {cache_idx if own else self.kv_from} holds no latent rows")
        q = torch.empty((T, H * (L + R)), dtype=torch.float32, device=h.device)
        latattn_prep(cfg, proj, 0, c_off, self.w["lat_norm"], self.w["inv_freq"], batch.positions, batch.cache_loc, lat if own else None, q)
        head_gemm(proj, D + R, self.w["ukT"], q, L + R)          # q_lat[h] = W_uk[h]^T q_unrotated[h]
        span = batch.max_kv_len if not self.window else min(batch.max_kv_len, self.window)
        if self.USE_MATRIX_CORES and lat.dtype == torch.bfloat16 and latattn_mfma_eligible(cfg):
            # workgroups of 64 (token, head) rows x key ranges, enough of them to fill the chip
            blocks = batch.B * ((batch.max_q_len * H + 63) // 64)
            nsplit = max(1, min(self.TARGET_WORKGROUPS // max(blocks, 1), (span + self.MFMA_KEYS_PER_SPLIT - 1) // self.MFMA_KEYS_PER_SPLIT))
            o_lat = latattn_mfma(cfg, q, lat, batch, self.w["sink"], nsplit=nsplit, out_dtype=self.compute_dtype)
        else:
            nsplit = max(1, min(self.TARGET_WORKGROUPS // max(T, 1), (span + self.KEYS_PER_SPLIT - 1) // self.KEYS_PER_SPLIT))
            o_lat = latattn_forward(cfg, q, lat, batch, self.w["sink"], nsplit=nsplit, out_dtype=self.compute_dtype)
        o = torch.empty((T, H * V), dtype=self.compute_dtype, device=h.device)
        head_gemm(o_lat, L, self.w["uv"], o, V)
        r_off = g_off + (H * V if self.gated else 0)
        if self.gated:
            o = sigmoid_gate_rows(o, proj[:, g_off:g_off + H * V], out_dtype=self.compute_dtype)
        return dense_gemm(o, self.w["o"]), (proj[:, r_off:] if rider is not None else None)
