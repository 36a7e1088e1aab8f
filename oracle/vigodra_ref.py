"""TEST INFRASTRUCTURE ONLY — plain, slow torch statement of the Vigodra design, one function per mechanism, evaluated on the
CPU in fp64 (or fp32).  It shares no code with ktransformers_amd: the product's operators, cache and kernels are compared
with it.  Whole sequences only: no cache, no batching, no chunking — a sequence is a list of token ids.

Notation: x[t] is the residual stream at position t (positions count from 0), W a weight stored [out, in] and applied as
W @ h, `P[name]` a tensor of the checkpoint, `cfg` the parsed config.json."""
from __future__ import annotations

import math

import torch

GLU_SIGMOID_SLOPE = 1.702        # fixed by the design: the feed-forward's gate is g * sigmoid(1.702 g)


def layer_norm(x, w, b, eps):
    mu = x.mean(dim=-1, keepdim=True)
    var = (x - mu).pow(2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps) * w


def causal_conv(u, w):
    """u [T, C], w [C, K]: y[t, c] = sum_j w[c, j] u[t - K + 1 + j, c] (the last column multiplies the current token), zeros before 0."""
    T, C = u.shape
    K = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance-bias table for distance n >= 0: the first rows / 2 distances have a row each, the rest share rows on a
    logarithmic scale that reaches the last row at distance `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def visible_matrix(T: int, size, keep_first: int = 0):
    """[i, j] true where position i sees position j: j <= i and (i - j < size or j < keep_first); size None: no window."""
    i, j = torch.arange(T).view(T, 1), torch.arange(T).view(1, T)
    near = torch.ones(T, T, dtype=torch.bool) if size is None else (i - j < size)
    return (j <= i) & (near | (j < keep_first))


def distance_bias_matrix(T: int, column, far: float):
    """[i, j] = column[bucket(i - j)] for j <= i (0 elsewhere): one head's learned bias by distance."""
    by_dist = torch.stack([column[distance_bucket(n, column.shape[0], far)] for n in range(T)])
    i, j = torch.arange(T).view(T, 1), torch.arange(T).view(1, T)
    return by_dist[(i - j).clamp(min=0)] * (j <= i)


def attention_core(q, k, v, scale, size=None, keep_first=0, rel=None, far=None, sink=None):
    """q [T, H, D], k [T, G, D], v [T, G, V] of ONE sequence -> [T, H, V]: softmax over the visible keys of scale q.k + rel[bucket(i - j), head]
    and, with sink [H], one extra score per head that only enlarges the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    see = visible_matrix(T, size, keep_first)
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale                            # [i, j]
        if rel is not None:
            s = s + distance_bias_matrix(T, rel[:, hd], far)
        s = s.masked_fill(~see, float("-inf"))
        if sink is not None:                                          # one more column whose weight is dropped
            s = torch.cat([s, sink[hd].expand(T, 1)], dim=1)
        w = torch.softmax(s, dim=1)[:, :T]
        out[:, hd] = w @ v[:, g]
    return out


def biased_window_attention(P, pre, c, h, eps):
    """Grouped-query attention without rotation: q, k, v = biased projections, each followed by a causal convolution over time;
    q and k are RMS-normed over their WHOLE projection (all heads at once) with a weight; score = scale q.k + table[bucket(i - j), head];
    a sliding window that also keeps the sequence's first tokens; one learned sink per head in the softmax's denominator."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    mask = c.get("mask") or {}
    size, keep = mask.get("size"), int(mask.get("keep_first") or 0)
    q = h @ P[pre + "q"].T + P[pre + "q.b"]
    k = h @ P[pre + "k"].T + P[pre + "k.b"]
    v = h @ P[pre + "v"].T + P[pre + "v.b"]
    if int(c.get("conv") or 0) > 0:
        q, k, v = causal_conv(q, P[pre + "q.conv"]), causal_conv(k, P[pre + "k.conv"]), causal_conv(v, P[pre + "v.conv"])
    q = rms_norm(q, P[pre + "q.norm"], eps).view(T, H, D)
    k = rms_norm(k, P[pre + "k.norm"], eps).view(T, G, D)
    v = v.view(T, G, V)
    out = attention_core(q, k, v, c["scale"], size, keep, P.get(pre + "rel"), c.get("bias_max"), P.get(pre + "sink"))
    return out.reshape(T, H * V) @ P[pre + "o"].T + P[pre + "o.b"]


def rotate_half(v, pos, base, dims):
    """v [T, ..., n]: entry i < dims / 2 of the last axis pairs with entry i + dims / 2; the pair turns by pos[t] * base^(-2i / dims)."""
    if dims == 0:
        return v
    out = v.clone()
    half = dims // 2
    i = torch.arange(half, dtype=v.dtype)
    ang = pos.to(v.dtype).view(-1, *([1] * (v.dim() - 1))) * torch.pow(torch.tensor(base, dtype=v.dtype), -2.0 * i / dims)
    cs, sn = torch.cos(ang), torch.sin(ang)
    a, b = v[..., :half], v[..., half:dims]
    out[..., :half] = a * cs - b * sn
    out[..., half:dims] = b * cs + a * sn
    return out


def latent_rows(P, pre, c, h, eps):
    """What a latent-attention layer keeps per token: the RMS-normed latent c [T, kv_rank] and the rotated key part [T, rot_dim]."""
    T = h.shape[0]
    L, R = c["kv_rank"], c["rot_dim"]
    d = h @ P[pre + "dkv"].T
    lat = rms_norm(d[:, :L], P[pre + "dkv.norm"], eps)
    rot = c.get("rot") or None
    kr = d[:, L:L + R]
    if rot:
        kr = rotate_half(kr, torch.arange(T), rot["base"], rot["dims"])
    return lat, kr


def latent_core(q_lat, rows, rank, scale, size=None):
    """The latent attention with the key product moved to the query side: q_lat [T, H, rank + rot] against the cached rows [T, rank + rot]
    (latent | rotated key part) of ONE sequence -> each head's softmax-weighted sum of the LATENTS [T, H, rank] (W_uv follows)."""
    T, H, _ = q_lat.shape
    see = visible_matrix(T, size, 0)
    out = torch.zeros(T, H, rank, dtype=q_lat.dtype)
    for hd in range(H):
        s = (q_lat[:, hd] @ rows.T) * scale
        out[:, hd] = torch.softmax(s.masked_fill(~see, float("-inf")), dim=1) @ rows[:, :rank]
    return out


def gated_latent_attention(P, pre, c, h, eps, shared=None):
    """Latent attention: keys and values of every head are products of one cached latent (plus one rotated key part all heads share);
    sliding window, ordinary softmax, heads multiplied by sigmoid(W_g h) before W_o.  `shared`: (latent, rotated key part) of the layer
    this one takes them from, instead of its own down projection."""
    T = h.shape[0]
    H, D, R, V, L = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    size = (c.get("mask") or {}).get("size")
    lat, kr = shared if shared is not None else latent_rows(P, pre, c, h, eps)
    q = (h @ P[pre + "q"].T).view(T, H, D + R)
    qn, qr = q[..., :D], q[..., D:]
    rot = c.get("rot") or None
    if rot:
        qr = rotate_half(qr, torch.arange(T), rot["base"], rot["dims"])
    kn = (lat @ P[pre + "uk"].T).view(T, H, D)
    v = (lat @ P[pre + "uv"].T).view(T, H, V)
    see = visible_matrix(T, size, 0)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * c["scale"]
        out[:, hd] = torch.softmax(s.masked_fill(~see, float("-inf")), dim=1) @ v[:, hd]
    o = out.reshape(T, H * V)
    if pre + "g" in P:
        o = o * torch.sigmoid(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T, (lat, kr)


def clamped_glu(P, pre, c, h):
    """W_down (g sigmoid(1.702 g) (u + 1)) with g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit)."""
    limit = c.get("limit")
    g, u = h @ P[pre + "gate"].T, h @ P[pre + "up"].T
    if limit is not None:
        g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
    return (g * torch.sigmoid(GLU_SIGMOID_SLOPE * g) * (u + 1.0)) @ P[pre + "down"].T


def depth_average(stack, w):
    """sum_j w[j] X_j over the embedding output X_0 and the results X_1 .. of the layers so far."""
    return sum(w[j] * stack[j] for j in range(len(stack)))


def forward(P, cfg, tokens, dtype=torch.float64, return_layers=False):
    """tokens: list of ids -> logits [T, vocab] (and, if asked, what every layer hands on [layers, T, width])."""
    P = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in P.items()}
    eps, alpha = cfg["norm"]["eps"], float(cfg.get("postln_alpha", 1.0))
    x = P["embed"][torch.tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    stack, kept, trail = [x], {}, []
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        c = L["mixer"]
        if L["type"] == "attention":
            y = biased_window_attention(P, pre + "mix.", c, x, eps)
        elif L["type"] == "latent_attention":
            src = c.get("kv_from")
            y, kept[i] = gated_latent_attention(P, pre + "mix.", c, x, eps, shared=None if src is None else kept[src])
        else:
            raise ValueError(L["type"])
        x = layer_norm(alpha * x + y, P[pre + "norm1"], P[pre + "norm1.b"], eps)
        if L.get("mlp") is not None:
            x = layer_norm(alpha * x + clamped_glu(P, pre + "mlp.", L["mlp"], x), P[pre + "norm2"], P[pre + "norm2.b"], eps)
        stack.append(x)
        if pre + "dwa" in P:
            x = depth_average(stack, P[pre + "dwa"])
        trail.append(x)
    logits = layer_norm(x, P["final.norm"], P["final.norm.b"], eps) @ P["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits


# ---- small configurations and random checkpoints for the tests ---------------------------------------------------------------------
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, keep_first=2, conv=3, bias_max=20, scale=None, mlp="dense"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "conv": conv, "bias_max": bias_max}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention", "mixer": m, "mlp": dense_mlp() if mlp == "dense" else mlp}


def latent_layer(heads=2, dim=8, rot_dim=8, vdim=12, kv_rank=16, window=10, base=10000.0, rot_dims=None, scale=None, kv_from=None, mlp="dense"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": dense_mlp() if mlp == "dense" else mlp}


def dense_mlp(ff=40, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def make_config(layers, width=32, vocab=61, eps=1e-5, alpha=1.7, scale=3.0):
    return {"architecture": "Vigodra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "postln_alpha": alpha, "layers": layers}


def random_checkpoint(cfg: dict, seed: int = 0, rel_rows: int = 8) -> dict:
    """Random bf16-representable weights with the checkpoint's tensor names for a config of the design."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    P = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W), "final.norm": vec(W, 1.0, 0.2), "final.norm.b": vec(W)}
    for li, layer in enumerate(cfg["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        P[p + "norm1"], P[p + "norm1.b"] = vec(W, 1.0, 0.2), vec(W)
        if layer["type"] == "attention":
            H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], int(m.get("conv") or 0)
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                P[p + f"mix.{n}"], P[p + f"mix.{n}.b"] = mat(rows, W), vec(rows, 0.0, 0.3)
                if K:
                    P[p + f"mix.{n}.conv"] = mat(rows, K, 0.6)
            P[p + "mix.q.norm"], P[p + "mix.k.norm"] = vec(H * D, 1.0, 0.3), vec(G * D, 1.0, 0.3)
            if m.get("bias_max") is not None:
                # (the far distance must lie beyond half the rows)
                P[p + "mix.rel"] = mat(rel_rows if m["bias_max"] > rel_rows // 2 else 2, H, 1.0)
            P[p + "mix.sink"] = vec(H, 0.0, 1.0)
            P[p + "mix.o"], P[p + "mix.o.b"] = mat(W, H * V), vec(W, 0.0, 0.3)
        else:
            H, D, R, V, L = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            P[p + "mix.q"] = mat(H * (D + R), W)
            if m.get("kv_from") is None:
                P[p + "mix.dkv"], P[p + "mix.dkv.norm"] = mat(L + R, W), vec(L, 1.0, 0.3)
            P[p + "mix.uk"], P[p + "mix.uv"] = mat(H * D, L), mat(H * V, L)
            P[p + "mix.g"], P[p + "mix.o"] = mat(H * V, W), mat(W, H * V)
        c = layer.get("mlp")
        if c:
            P[p + "norm2"], P[p + "norm2.b"] = vec(W, 1.0, 0.2), vec(W)
            P[p + "mlp.gate"], P[p + "mlp.up"], P[p + "mlp.down"] = mat(c["ff"], W, 2.0 / math.sqrt(W)), mat(c["ff"], W, 2.0 / math.sqrt(W)), mat(W, c["ff"])
        P[p + "dwa"] = (torch.randn(li + 2, generator=g) * 0.5 + torch.nn.functional.one_hot(torch.tensor(li + 1), li + 2)).to(torch.bfloat16)
    return P


def as_double(P: dict) -> dict:
    return {k: (v.double() if v.is_floating_point() else v) for k, v in P.items()}
