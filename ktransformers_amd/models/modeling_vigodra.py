"""Module skeleton of Vigodra — a POST-normed decoder with an fp32 residual stream: every sublayer reads the residual x itself and
x <- layer_norm(alpha * x + sublayer(x)) (weight and bias, a residual scaled by `postln_alpha`); behind every layer a depth-weighted
average hands on sum_j w[j] X_j over the embedding output X_0 and the results X_1 .. of all layers so far.  A layer mixes tokens either
with a grouped-query attention without rotation (biased projections followed by a short causal convolution over time, RMS norms over the
whole q and k projections, a learned bias by bucketed distance, a sliding window that keeps the sequence's first tokens, a learned sink
per head) or with a sliding-window latent attention (rotate-half positions on a shared key part, ordinary softmax, a sigmoid output
gate), whose cached latent rows a later layer may re-use (`kv_from`).  The feed-forward is a GLU whose halves are bounded before they meet.

Like the other skeletons of this package it only holds the structure the optimize rules inject into (optimize_rules/Vigodra.yaml) and
the glue (which launch a sublayer's output joins the residual in); every module that does arithmetic is a leaf that raises until an
operator replaces it.  Module paths equal the checkpoint's tensor prefixes:

    embed | l<i>.{mix,norm1,mlp,norm2,dwa} | final.norm | head

config.json: {"architecture": "Vigodra", "width", "vocab", "norm": {"eps"}, "embedding": {"scale"}, "postln_alpha",
"layers": [{"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "conv", "bias_max",
                                           "mask": {"size", "keep_first"} | null}, "mlp": ...} |
           {"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot": {"base", "dims"},
                                                  "mask": {"size"} | null, "kv_from": j (optional)}, "mlp": ...}],
 mlp: null | {"kind": "dense", "ff", "limit"}}.
Sizes and the constants listed there come from the file (the number of distance-bias rows from the tensor's shape); what the design
fixes is a constant here."""
from __future__ import annotations

import json
import os
from types import SimpleNamespace

import torch
from torch import nn

from ktransformers_amd.models.modeling_deepseek import _Leaf

# fixed by the design
GLU_SIGMOID_SLOPE = 1.702      # the feed-forward's gate is g * sigmoid(1.702 g)
GLU_UP_SHIFT = 1.0             # ... times (u + 1)
MIXER_TYPES = ("attention", "latent_attention")
MLP_KINDS = ("dense",)


def make_vigodra_config(d: dict | str, compute_dtype=torch.bfloat16) -> SimpleNamespace:
    """config.json (a dict or a path) -> the namespace the skeleton and the operators read."""
    if isinstance(d, str):
        with open(os.path.join(d, "config.json") if os.path.isdir(d) else d, encoding="utf-8") as f:
            d = json.load(f)
    if d.get("architecture") != "Vigodra":
        raise ValueError(f"not a Vigodra config: architecture = {d.get('architecture')!r}")
    layers = list(d["layers"])
    for i, L in enumerate(layers):
        if L.get("type") not in MIXER_TYPES:
            raise ValueError(f"layer {i}: unknown layer type {L.get('type')!r}")
        m = L["mixer"]
        if L["type"] == "attention":
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads ({m['heads']}) must be a multiple of kv_heads ({m['kv_heads']})")
        else:
            rot = m.get("rot") or None
            if rot and (rot["dims"] % 2 or rot["dims"] > m["rot_dim"]):
                raise ValueError(f"layer {i}: rot.dims ({rot['dims']}) must be even and at most rot_dim ({m['rot_dim']})")
            src = m.get("kv_from")
            if src is not None:
                s = layers[src]["mixer"] if 0 <= src < i and layers[src]["type"] == "latent_attention" else None
                if s is None or s.get("kv_from") is not None or any(s.get(k) != m.get(k) for k in ("kv_rank", "rot_dim", "rot")):
                    raise ValueError(f"layer {i}: kv_from ({src}) must name an earlier latent-attention layer with a down projection of its "
                                     "own and equal kv_rank, rot_dim and rotation")
        c = L.get("mlp")
        if c is not None and c.get("kind") not in MLP_KINDS:
            raise ValueError(f"layer {i}: unknown feed-forward kind {c.get('kind')!r}")
    return SimpleNamespace(architectures=["Vigodra"], width=int(d["width"]), vocab=int(d["vocab"]), eps=float(d["norm"]["eps"]),
                           embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)), alpha=float(d.get("postln_alpha", 1.0)),
                           layers=layers, num_hidden_layers=len(layers), vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                           compute_dtype=compute_dtype, max_position_embeddings=None, raw=d)


def vigodra_layer_specs(config) -> list:
    """What KHybridCache needs, one entry per layer: paged key / value rows plus the convolution's state for an attention layer, paged
    latent rows for a latent-attention layer with a down projection of its own, nothing for one that reads another layer's rows."""
    specs = []
    for L in config.layers:
        m = L["mixer"]
        if L["type"] == "attention":
            H, G, D, V = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            spec = {"kv": (G, D, V)}
            if int(m.get("conv") or 0) > 1:
                spec["conv"] = (H * D + G * (D + V), int(m["conv"]))
        else:
            spec = {} if m.get("kv_from") is not None else {"latent": int(m["kv_rank"]) + int(m["rot_dim"])}
        specs.append(spec)
    return specs


class VigodraEmbedding(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.vocab, self.width, self.scale = config.vocab, config.width, config.embed_scale


class VigodraNorm(_Leaf):
    def __init__(self, width, eps):
        super().__init__()
        self.width, self.eps = width, eps


class VigodraDepthAverage(_Leaf):
    def __init__(self, levels):
        super().__init__()
        self.levels = levels


class VigodraAttention(_Leaf):
    """Grouped-query attention, no rotation: the options KWindowGQAttention reads."""

    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps = config.width, config.eps
        self.heads, self.kv_heads, self.dim, self.vdim = (int(c[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.scale = float(c["scale"])
        mask = c.get("mask") or {}
        self.window = int(mask.get("size") or 0)
        self.keep_first = int(mask.get("keep_first") or 0) if self.window else 0
        self.rot_dims, self.rot_base, self.rot_values, self.qk_norm, self.sink_score = 0, 1.0, False, False, None
        self.qkv_bias = self.out_bias_on = self.proj_norm = True
        self.conv_taps = int(c.get("conv") or 0)
        self.sink = "learned"
        self.dist_far = float(c["bias_max"]) if c.get("bias_max") is not None else None


class VigodraLatentAttention(_Leaf):
    """Sliding-window latent attention: the options KLatentWindowAttention reads."""

    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps = config.width, config.eps
        self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = (int(c[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale = float(c["scale"])
        self.window = int((c.get("mask") or {}).get("size") or 0)
        rot = c.get("rot") or None
        self.rot_dims, self.rot_base = (int(rot["dims"]), float(rot["base"])) if rot else (0, 1.0)
        self.rot_half, self.has_sink, self.gated = True, False, True
        self.kv_from = None if c.get("kv_from") is None else int(c["kv_from"])


class VigodraMLP(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.ff = config.width, int(c["ff"])
        self.limit = None if c.get("limit") is None else float(c["limit"])
        self.slope, self.up_shift = GLU_SIGMOID_SLOPE, GLU_UP_SHIFT


class VigodraLayer(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        L = config.layers[layer_idx]
        self.alpha, self.level = config.alpha, layer_idx + 1
        self.mix = VigodraAttention(config, L["mixer"]) if L["type"] == "attention" else VigodraLatentAttention(config, L["mixer"])
        self.latent = L["type"] == "latent_attention"
        self.norm1 = VigodraNorm(config.width, config.eps)
        self.mlp = None if L.get("mlp") is None else VigodraMLP(config, L["mlp"])
        if self.mlp is not None:
            self.norm2 = VigodraNorm(config.width, config.eps)
        self.dwa = VigodraDepthAverage(layer_idx + 2)

    def forward(self, x_in, x, h, stack, batch, cache, cache_idx, lp_dtype, last: bool = False):
        """x_in fp32 [T, W]: what the layer reads (x itself, or level 0 of the stack for the first layer); h = x_in in the compute type.
        x <- norm1(alpha x_in + mix(h)); x <- norm2(alpha x + mlp(x)); level `level` of the stack <- x; x <- the depth-weighted average.
        Each step is one launch behind the sublayer's products.  Returns x in the compute type (what the next layer's products read)."""
        if self.latent:
            y, _ = self.mix(h, batch, cache, cache_idx)
            ybias = None
        else:
            y = self.mix(h, batch, cache, cache_idx)
            ybias = self.mix.out_bias
        closing = dict(stack=stack, level=self.level, depth=self.dwa, lp_dtype=None if last else lp_dtype)
        if self.mlp is None:
            return self.norm1.post_mix(x_in, x, y=y, ybias=ybias, alpha=self.alpha, **closing)
        h = self.norm1.post_mix(x_in, x, y=y, ybias=ybias, alpha=self.alpha, lp_dtype=lp_dtype)
        return self.norm2.post_mix(x, x, y=self.mlp(h), alpha=self.alpha, **closing)


class _Final(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.norm = VigodraNorm(config.width, config.eps)


class VigodraHead(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.in_features, self.out_features = config.width, config.vocab


class VigodraForCausalLM(nn.Module):
    """forward(input_ids, position_ids, past_key_values, cache_position, batch=, logits_rows=, last_token_only=) -> fp32 logits.

    With `batch` (a ForwardBatch planned by the KHybridCache in `past_key_values`): input_ids is the flattened token list of the
    step and the result is [len(logits_rows) or T, vocab].  Without it, the call is the single-sequence form the generation loop
    uses (util/generate.py): input_ids [1, T] at position_ids [1, T]; the result is [1, T or 1, vocab]."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed = VigodraEmbedding(config)
        for i in range(config.num_hidden_layers):
            self.add_module(f"l{i}", VigodraLayer(config, i))
        self.final = _Final(config)
        self.head = VigodraHead(config)

    def forward(self, input_ids=None, position_ids=None, past_key_values=None, cache_position=None, batch=None, logits_rows=None,
                last_token_only: bool = False, return_layers: bool = False):
        cache = past_key_values
        single = batch is None
        if single:
            batch = cache.single_request_batch(position_ids)
            if last_token_only and batch.T > 1:
                logits_rows = torch.tensor([batch.T - 1], dtype=torch.int32, device=cache.device)
        tokens = input_ids.reshape(-1).to(torch.int32)
        n, W, cd = self.config.num_hidden_layers, self.config.width, self.config.compute_dtype
        T = tokens.numel()
        # level 0 = the embedding output, level i + 1 = layer i's result: what the depth-weighted averages sum over
        stack = torch.empty((n + 1, T, W), dtype=torch.float32, device=tokens.device)
        x0 = self.embed(tokens, batch.positions, out=stack[0])
        x = torch.empty((T, W), dtype=torch.float32, device=tokens.device)
        h = x0 if cd == torch.float32 else x0.to(cd)
        trail = []
        for i in range(n):
            h = getattr(self, f"l{i}")(x0 if i == 0 else x, x, h, stack, batch, cache, i, cd, last=i == n - 1)
            if return_layers:
                trail.append(x.clone())
        h = self.final.norm(x if n else x0, rows=logits_rows, out_dtype=cd)
        logits = self.head(h)
        if single:
            logits = logits.unsqueeze(0)
        return (logits, torch.stack(trail)) if return_layers else logits
