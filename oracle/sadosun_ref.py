"""TEST INFRASTRUCTURE ONLY — plain, slow torch statement of the Sadosun design, one function per mechanism, evaluated on the
CPU in fp64 (or fp32).  It shares no code with ktransformers_amd: the product's operators, cache and kernels are compared
with it.  Whole sequences only: no cache, no batching, no chunking — a sequence is a list of token ids.

Notation: x[t] is the residual stream at position t (positions count from 0), W a weight stored [out, in] and applied as
W @ h, `P[name]` a tensor of the checkpoint, `cfg` the parsed config.json."""
from __future__ import annotations

import math

import torch

ROUTER_SUM_EPS = 1e-20


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is ONE number for all coordinates."""
    return unit_rms(x, eps) * g


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x, w):
    """x [T, C], w [C, K]: y[t, c] = sum_j w[c, j] x[t - K + 1 + j, c] (the last column multiplies the current token), zeros before 0."""
    T, C = x.shape
    K = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def input_conv(h, w):
    """What a sublayer reads: h + conv(h)."""
    return h + causal_conv(h, w)


def turn_pairs(v, pos, base, dims, sign=1.0):
    """v [T, ..., n]: the first `dims` entries of the last axis as pairs (2i, 2i + 1) turned by sign * pos[t] * base^(-2i / dims)."""
    if dims == 0:
        return v
    out = v.clone()
    i = torch.arange(dims // 2, dtype=v.dtype)
    ang = sign * pos.to(v.dtype).view(-1, *([1] * (v.dim() - 1))) * torch.pow(torch.tensor(base, dtype=v.dtype), -2.0 * i / dims)
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def attention_mixer(P, pre, c, h, eps):
    """Grouped-query sliding-window attention: partially rotated, unit-RMS q and k; values turned by their own position and the
    result turned back by the query's; one extra unit (a sink of score 0 without a value) in the softmax's denominator."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    rot = c.get("rot") or None
    window = (c.get("mask") or {}).get("size")
    pos = torch.arange(T)
    q = (h @ P[pre + "q"].T).view(T, H, D)
    k = (h @ P[pre + "k"].T).view(T, G, D)
    v = (h @ P[pre + "v"].T).view(T, G, V)
    if rot:
        q = turn_pairs(q, pos, rot["base"], rot["dims"])
        k = turn_pairs(k, pos, rot["base"], rot["dims"])
        v = turn_pairs(v, pos, rot["base"], V)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * c["scale"]                        # [i, j]
        d = pos.view(-1, 1) - pos.view(1, -1)
        ok = d >= 0
        if window:
            ok = ok & (d < window)
        e = torch.where(ok, torch.exp(s), torch.zeros_like(s))
        p = e / (1.0 + e.sum(dim=1, keepdim=True))
        out[:, hd] = p @ v[:, g]
    if rot:
        out = turn_pairs(out, pos, rot["base"], V, sign=-1.0)
    return out.reshape(T, H * V) @ P[pre + "o"].T


def mamba_mixer(P, pre, c, h):
    """Selective scan: per channel c and state n, S <- exp(dt A) S + dt x B;  y = S . C + D x;  gated by silu(z)."""
    T = h.shape[0]
    inner, N, R = c["inner"], c["state"], c["dt_rank"]
    xz = h @ P[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, P[pre + "conv"]) + P[pre + "conv.b"])
    xp = x @ P[pre + "x"].T
    dt, B, C = xp[:, :R], xp[:, R:R + N], xp[:, R + N:]
    dt = softplus(dt @ P[pre + "dt"].T + P[pre + "dt.b"])              # [T, inner]
    A = -torch.exp(P[pre + "A_log"])                                   # [inner, N]
    S = torch.zeros(inner, N, dtype=h.dtype)
    y = torch.zeros(T, inner, dtype=h.dtype)
    for t in range(T):
        S = torch.exp(dt[t].view(-1, 1) * A) * S + (dt[t] * x[t]).view(-1, 1) * B[t].view(1, -1)
        y[t] = S @ C[t] + P[pre + "D"] * x[t]
    return (y * silu(z)) @ P[pre + "o"].T


def route(P, pre, c, h):
    """-> (chosen expert indices [T, top], weights [T, top]).  Scores = softmax over ALL router outputs; the choice adds a
    correction per expert, the weights do not; weights are the chosen scores over their sum."""
    z = h @ P[pre + "router"].T
    s = torch.softmax(z, dim=-1)
    choice = s + P[pre + "correction"] if pre + "correction" in P else s
    idx = torch.topk(choice, c["router"]["top"], dim=-1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(dim=-1, keepdim=True) + ROUTER_SUM_EPS)


def moe_ff(P, pre, c, h):
    """Mixture of relu^2 experts; the LAST `identity` router outputs stand for experts that return their input."""
    E = c["router"]["experts"]
    idx, w = route(P, pre, c, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            if e >= E:
                y = h[t]
            else:
                y = P[f"{pre}e{e}.down"] @ torch.relu(P[f"{pre}e{e}.up"] @ h[t]).pow(2)
            out[t] += w[t, k] * y
    return out


def side_input(P, pre, x, e, eps):
    """The per-layer token input: y = W_proj (gelu(W_gate x) * e);  returns y / rms(y) * w (what is added to x)."""
    y = (gelu_tanh(x @ P[pre + "gate"].T) * e) @ P[pre + "proj"].T
    return unit_rms(y, eps) * P[pre + "norm"]


def forward(P, cfg, tokens, dtype=torch.float64, return_layers=False):
    """tokens: list of ids -> logits [T, vocab] (and the residual stream after every layer, [layers, T, width])."""
    P = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in P.items()}
    tok = torch.tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x = P["embed"][tok] * cfg["embedding"]["scale"]
    canon = (cfg.get("canon") or {}).get("taps")
    side = (cfg.get("token_side") or {}).get("dim")
    trail = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, P[p + "norm1"], eps)
        if canon:
            h = input_conv(h, P[p + "canon1"])
        if L["type"] == "attention":
            x = x + attention_mixer(P, p + "mix.", L["mixer"], h, eps)
        elif L["type"] == "mamba1":
            x = x + mamba_mixer(P, p + "mix.", L["mixer"], h)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            h = scalar_norm(x, P[p + "norm2"], eps)
            if canon:
                h = input_conv(h, P[p + "canon2"])
            x = x + moe_ff(P, p + "mlp.", L["mlp"], h)
        if side:
            x = x + side_input(P, p + "side.", x, P["side.embed"][tok][:, i * side:(i + 1) * side], eps)
        trail.append(x.clone())
    logits = scalar_norm(x, P["final.norm"], eps) @ P["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits


# ---- small configurations and random checkpoints for the tests ---------------------------------------------------------------------
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, rot_dims=None, base=10000.0, scale=None, rot=True, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if rot:
        m["rot"] = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def scan_layer(inner=48, state=8, dt_rank=4, conv=3, mlp=None):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}, "mlp": mlp}


def moe_mlp(experts=5, top=2, identity=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity}}


def make_config(layers, width=32, vocab=61, eps=1e-5, taps=3, side=6, scale=4.0):
    cfg = {"architecture": "Sadosun", "width": width, "vocab": vocab, "norm": {"eps": eps}, "embedding": {"scale": scale}, "layers": layers}
    if taps:
        cfg["canon"] = {"taps": taps}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def random_checkpoint(cfg: dict, seed: int = 0) -> dict:
    """Random bf16-representable weights with the checkpoint's tensor names for a config of the design."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    def one(mean=1.0, s=0.2):
        return (mean + torch.randn((), generator=g) * s).to(torch.bfloat16)

    taps = (cfg.get("canon") or {}).get("taps")
    side = (cfg.get("token_side") or {}).get("dim")
    P = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W), "final.norm": one()}
    if side:
        P["side.embed"] = mat(cfg["vocab"], side * len(cfg["layers"]), 1.0)
    for li, layer in enumerate(cfg["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        P[p + "norm1"] = one()
        if taps:
            P[p + "canon1"] = mat(W, taps, 0.4)
        if layer["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            P[p + "mix.q"], P[p + "mix.k"], P[p + "mix.v"] = mat(H * D, W), mat(G * D, W), mat(G * V, W)
            P[p + "mix.o"] = mat(W, H * V)
        else:
            I, N, R, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            P[p + "mix.in"], P[p + "mix.conv"], P[p + "mix.conv.b"] = mat(2 * I, W), mat(I, K, 0.5), vec(I)
            P[p + "mix.x"], P[p + "mix.dt"], P[p + "mix.dt.b"] = mat(R + 2 * N, I), mat(I, R), vec(I, -1.0, 1.0)
            P[p + "mix.A_log"], P[p + "mix.D"], P[p + "mix.o"] = mat(I, N, 0.7), vec(I, 1.0, 0.3), mat(W, I)
        c = layer.get("mlp")
        if c:
            P[p + "norm2"] = one()
            if taps:
                P[p + "canon2"] = mat(W, taps, 0.4)
            E, ID, F = c["router"]["experts"], c["router"].get("identity") or 0, c["expert"]["ff"]
            P[p + "mlp.router"], P[p + "mlp.correction"] = mat(E + ID, W, 2.0 / math.sqrt(W)), vec(E + ID, 0.0, 0.05)
            for e in range(E):
                P[p + f"mlp.e{e}.up"], P[p + f"mlp.e{e}.down"] = mat(F, W), mat(W, F)
        if side:
            P[p + "side.gate"], P[p + "side.proj"], P[p + "side.norm"] = mat(side, W, 0.5 / math.sqrt(W)), mat(W, side), vec(W, 0.7, 0.2)
    return P


def as_double(P: dict) -> dict:
    return {k: (v.double() if v.is_floating_point() else v) for k, v in P.items()}
