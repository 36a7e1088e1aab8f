"""Module skeleton of Sadosun — a pre-normed decoder with an fp32 residual stream whose layers mix tokens either with a grouped-query
sliding-window attention (partly rotated unit-RMS queries and keys, values rotated relative to the query, a sink of score 0 in the
softmax) or with a selective scan (Mamba), behind RMS norms whose weight is one number and a causal convolution over time on what each
sublayer reads; the feed-forward is a softmax-routed mixture of relu^2 experts some of whose router outputs stand for the identity;
after it every layer adds an input looked up by token.

Like the other skeletons of this package it only holds the structure the optimize rules inject into (optimize_rules/Sadosun.yaml) and
the glue (the layer's residual arrangement: what a sublayer produced joins the residual in the launch that norms it for the next one);
every module that does arithmetic is a leaf that raises until an operator replaces it.  Module paths equal the checkpoint's tensor
prefixes:

    embed | side | l<i>.{norm1,canon1,mix,norm2,canon2,mlp,side} | final.norm | head

config.json: {"architecture": "Sadosun", "width", "vocab", "norm": {"eps"}, "embedding": {"scale"}, "canon": {"taps"} | null,
"token_side": {"dim"} | null,
"layers": [{"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"} | null,
                                           "rot": {"base", "dims"} | null}, "mlp": ...} |
           {"type": "mamba1", "mixer": {"inner", "state", "dt_rank", "conv"}, "mlp": ...}],
 mlp: null | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "identity"}}}.
Sizes and the constants listed there come from the file; what the design fixes is a constant here."""
from __future__ import annotations

import json
import os
from types import SimpleNamespace

import torch
from torch import nn

from ktransformers_amd.models.modeling_deepseek import _Leaf

# fixed by the design
ROUTER_SUM_EPS = 1e-20         # chosen scores / (their sum + 1e-20)
SINK_SCORE = 0.0               # the softmax's denominator holds exp(0) beside the keys' terms
MIXER_TYPES = ("attention", "mamba1")
MLP_KINDS = ("moe",)


def make_sadosun_config(d: dict | str, compute_dtype=torch.bfloat16) -> SimpleNamespace:
    """config.json (a dict or a path) -> the namespace the skeleton and the operators read."""
    if isinstance(d, str):
        with open(os.path.join(d, "config.json") if os.path.isdir(d) else d, encoding="utf-8") as f:
            d = json.load(f)
    if d.get("architecture") != "Sadosun":
        raise ValueError(f"not a Sadosun config: architecture = {d.get('architecture')!r}")
    layers = list(d["layers"])
    for i, L in enumerate(layers):
        if L.get("type") not in MIXER_TYPES:
            raise ValueError(f"layer {i}: unknown layer type {L.get('type')!r}")
        m = L["mixer"]
        if L["type"] == "attention":
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: heads ({m['heads']}) must be a multiple of kv_heads ({m['kv_heads']})")
            rot = m.get("rot")
            if rot and (rot["dims"] % 2 or rot["dims"] > m["dim"] or m["vdim"] % 2):
                raise ValueError(f"layer {i}: rot.dims ({rot['dims']}) must be even and at most dim ({m['dim']}), vdim ({m['vdim']}) even")
        if L.get("mlp") is not None:
            c = L["mlp"]
            if c.get("kind") not in MLP_KINDS:
                raise ValueError(f"layer {i}: unknown feed-forward kind {c.get('kind')!r}")
            r = c["router"]
            if not 0 < r["top"] <= r["experts"] + int(r.get("identity") or 0):
                raise ValueError(f"layer {i}: top ({r['top']}) must lie in 1 .. experts + identity")
    canon = int((d.get("canon") or {}).get("taps") or 0)
    side = int((d.get("token_side") or {}).get("dim") or 0)
    return SimpleNamespace(architectures=["Sadosun"], width=int(d["width"]), vocab=int(d["vocab"]), eps=float(d["norm"]["eps"]),
                           embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)), canon_taps=canon, side_dim=side, layers=layers,
                           num_hidden_layers=len(layers), vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                           compute_dtype=compute_dtype, max_position_embeddings=None, raw=d)


def sadosun_layer_specs(config) -> list:
    """What KHybridCache needs, one entry per layer: the mixer's cache or state plus the input convolutions' state of both sublayers."""
    specs = []
    pre = (config.width, config.canon_taps) if config.canon_taps > 1 else None
    for L in config.layers:
        m = L["mixer"]
        if L["type"] == "attention":
            spec = {"kv": (int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]))}
        else:
            spec = {"ssm": (int(m["inner"]), int(m["state"])), "conv": (int(m["inner"]), int(m.get("conv", 1)))}
        spec["pre"] = [pre, pre if L.get("mlp") is not None else None]
        specs.append(spec)
    return specs


class SadosunEmbedding(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.vocab, self.width, self.scale = config.vocab, config.width, config.embed_scale


class SadosunSideTable(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.vocab, self.dim, self.layers = config.vocab, config.side_dim, config.num_hidden_layers


class SadosunSideInput(_Leaf):
    def __init__(self, config, layer_idx):
        super().__init__()
        self.width, self.dim, self.layer_idx, self.eps = config.width, config.side_dim, layer_idx, config.eps


class SadosunNorm(_Leaf):
    def __init__(self, width, eps):
        super().__init__()
        self.width, self.eps = width, eps


class SadosunInputConv(_Leaf):
    def __init__(self, width, taps):
        super().__init__()
        self.width, self.taps = width, taps


class SadosunAttention(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps = config.width, config.eps
        self.heads, self.kv_heads, self.dim, self.vdim = (int(c[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.scale = float(c["scale"])
        self.window = int((c.get("mask") or {}).get("size") or 0)
        rot = c.get("rot") or None
        self.rot_dims, self.rot_base = (int(rot["dims"]), float(rot["base"])) if rot else (0, 1.0)
        self.rot_values = bool(rot)          # values turn with their position whenever the layer rotates at all
        self.qk_norm, self.sink_score = True, SINK_SCORE


class SadosunScanMixer(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width = config.width
        self.inner, self.state, self.dt_rank, self.taps = int(c["inner"]), int(c["state"]), int(c["dt_rank"]), int(c.get("conv", 1))


class SadosunMoE(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width = config.width
        r = c["router"]
        self.experts, self.top, self.identity = int(r["experts"]), int(r["top"]), int(r.get("identity") or 0)
        self.sum_eps = ROUTER_SUM_EPS
        self.ff = int(c["expert"]["ff"])


class SadosunLayer(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        L = config.layers[layer_idx]
        W, eps, taps = config.width, config.eps, config.canon_taps
        self.norm1 = SadosunNorm(W, eps)
        self.canon1 = SadosunInputConv(W, taps) if taps else None
        self.mix = SadosunAttention(config, L["mixer"]) if L["type"] == "attention" else SadosunScanMixer(config, L["mixer"])
        self.mlp = None if L.get("mlp") is None else SadosunMoE(config, L["mlp"])
        if self.mlp is not None:
            self.norm2 = SadosunNorm(W, eps)
            self.canon2 = SadosunInputConv(W, taps) if taps else None
        self.side = SadosunSideInput(config, layer_idx) if config.side_dim else None

    def pre(self, x, batch, cache, cache_idx, **pending):
        """What the mixer reads: conv1(norm1(x)) after `pending` (a sublayer's output not yet added) has joined x — one or two launches."""
        st = cache.pre_conv[cache_idx][0] if self.canon1 is not None else None
        return self.norm1(x, batch, conv=self.canon1, conv_state=st, **pending)

    def forward(self, x, tokens, batch, cache, cache_idx, h, side_table=None, following=None, following_idx=None):
        """x <- x + mix(h), h = conv1(norm1(x)) (given);  x <- x + mlp(conv2(norm2(x)));  x <- x + unit_rms(side(x)) * w.  x is the fp32
        residual and is updated in place.  Each sublayer's output joins x in the launch that norms x for the next sublayer; the last
        one joins in `following.pre` (the next layer's) when there is one.  Returns (x, what the next layer's mixer reads or None)."""
        from ktransformers_amd.operators.layernorm import residual_add
        pending = {"y": self.mix(h, batch, cache, cache_idx)}
        if self.mlp is not None:
            st = cache.pre_conv[cache_idx][1] if self.canon2 is not None else None
            h = self.norm2(x, batch, conv=self.canon2, conv_state=st, **pending)
            rows, pair_pos, idx, wts, n_real, h_in = self.mlp(h)
            pending = {"moe": (rows, pair_pos, idx, wts, n_real, h_in)}
        if self.side is not None:
            residual_add(x, **pending)
            pending = {"y": self.side(x, tokens, side_table), "y_norm": self.side.y_norm}
        if following is not None:
            return x, following.pre(x, batch, cache, following_idx, **pending)
        residual_add(x, **pending)
        return x, None


class _Final(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.norm = SadosunNorm(config.width, config.eps)


class SadosunHead(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.in_features, self.out_features = config.width, config.vocab


class SadosunForCausalLM(nn.Module):
    """forward(input_ids, position_ids, past_key_values, cache_position, batch=, logits_rows=, last_token_only=) -> fp32 logits.

    With `batch` (a ForwardBatch planned by the KHybridCache in `past_key_values`): input_ids is the flattened token list of the
    step and the result is [len(logits_rows) or T, vocab].  Without it, the call is the single-sequence form the generation loop
    uses (util/generate.py): input_ids [1, T] at position_ids [1, T]; the result is [1, T or 1, vocab]."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed = SadosunEmbedding(config)
        if config.side_dim:
            self.side = SadosunSideTable(config)
        for i in range(config.num_hidden_layers):
            self.add_module(f"l{i}", SadosunLayer(config, i))
        self.final = _Final(config)
        self.head = SadosunHead(config)

    def forward(self, input_ids=None, position_ids=None, past_key_values=None, cache_position=None, batch=None, logits_rows=None,
                last_token_only: bool = False, return_layers: bool = False):
        cache = past_key_values
        single = batch is None
        if single:
            batch = cache.single_request_batch(position_ids)
            if last_token_only and batch.T > 1:
                logits_rows = torch.tensor([batch.T - 1], dtype=torch.int32, device=cache.device)
        tokens = input_ids.reshape(-1).to(torch.int32)
        x = self.embed(tokens, batch.positions)
        table = self.side() if self.config.side_dim else None
        n = self.config.num_hidden_layers
        layers = [getattr(self, f"l{i}") for i in range(n)]
        trail = []
        h = layers[0].pre(x, batch, cache, 0)
        for i, layer in enumerate(layers):
            nxt = layers[i + 1] if i + 1 < n else None
            x, h = layer(x, tokens, batch, cache, i, h, side_table=table, following=nxt, following_idx=i + 1)
            if return_layers:
                trail.append(x.clone())
        h = self.final.norm(x, rows=logits_rows, out_dtype=self.config.compute_dtype)
        logits = self.head(h)
        if single:
            logits = logits.unsqueeze(0)
        return (logits, torch.stack(trail)) if return_layers else logits
