"""ctypes binding of include/ktx_hyb.h — the hybrid-decoder kernels (layer norm with bias, the gated post-normed residual update,
PolyNorm, the gated delta rule over state slots, sliding-window softmax attention with a sink over a paged latent cache, the sigmoid
top-k router, the expert sort and the grouped GEMM).  Same library and calling rules as ktransformers_amd._native_seq: device
pointers and the caller's current HIP stream cross the boundary, every call is graph-capturable, there is no CPU fallback."""
from __future__ import annotations

import ctypes as C

import torch

from ktransformers_amd._native_seq import SEQ_DTYPE, KtxError, _seq_dev, _stream_ptr, check, lib


class _DeltaConfig(C.Structure):     # include/ktx_hyb.h: ktx_delta_config
    _fields_ = [("heads", C.c_int32), ("kv_heads", C.c_int32), ("dim", C.c_int32), ("vdim", C.c_int32), ("taps", C.c_int32),
                ("unit_eps", C.c_float)]


class _PostNormArgs(C.Structure):    # include/ktx_hyb.h: ktx_postnorm_args
    _fields_ = [("y", C.c_void_p), ("ldy", C.c_int64), ("ybias", C.c_void_p), ("alpha", C.c_float), ("w", C.c_void_p), ("b", C.c_void_p),
                ("eps", C.c_float), ("stack", C.c_void_p), ("stack_stride", C.c_int64), ("level", C.c_int32), ("dwa", C.c_void_p),
                ("out_lp", C.c_void_p), ("out_dtype", C.c_int32)]


class _LatAttnConfig(C.Structure):   # include/ktx_hyb.h: ktx_latattn_config
    _fields_ = [("heads", C.c_int32), ("dim", C.c_int32), ("rot_dim", C.c_int32), ("vdim", C.c_int32), ("kv_rank", C.c_int32),
                ("rot_dims", C.c_int32), ("scale", C.c_float), ("window", C.c_int32), ("eps", C.c_float), ("page_size", C.c_int32),
                ("cache_dtype", C.c_int32), ("rot_half", C.c_int32)]


_P, _I, _L, _F = C.c_void_p, C.c_int, C.c_int64, C.c_float
if not hasattr(lib, "ktx_grouped_gemm"):
    raise ImportError("the loaded kernel library predates include/ktx_hyb.h: rebuild with `python -m ktransformers_amd.build [--seq]`")
lib.ktx_rows_add.argtypes = [_I, _I, _P, _P, _P, _P]
lib.ktx_layer_norm.argtypes = [_I, _I, _P, _P, _P, _F, _P, _P, _I, _P]
lib.ktx_gated_norm_add.argtypes = [_I, _I, _P, _L, _P, _P, _P, _P, _I, _P, _L, _P, _P, _P, _F, _P, _P, _P, _F, _P, _I, _P]
lib.ktx_poly_norm.argtypes = [_I, _I, _P, _L, _P, _P, _F, _P, _I, _P]
lib.ktx_silu_mul_rows.argtypes = [_I, _I, _P, _L, _P, _I, _P]
lib.ktx_postnorm_mix.argtypes = [_I, _I, _P, _P, C.POINTER(_PostNormArgs), _P]
lib.ktx_glu_clamp_rows.argtypes = [_I, _I, _P, _L, _F, _F, _F, _I, _P, _I, _P]
lib.ktx_sigmoid_gate_rows.argtypes = [_I, _I, _P, _I, _P, _L, _P, _I, _P]
lib.ktx_head_gate_norm.argtypes = [_I, _I, _I, _F, _P, _P, _L, _P, _I, _I, _P, _I, _P]
lib.ktx_delta_prep.argtypes = [C.POINTER(_DeltaConfig), _I, _I, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P]
lib.ktx_delta_forward.argtypes = [C.POINTER(_DeltaConfig), _I, _P, _P, _P, _P, _P, _P, _P, _P]
lib.ktx_latattn_prep.argtypes = [C.POINTER(_LatAttnConfig), _I, _P, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P]
lib.ktx_latattn_forward.argtypes = [C.POINTER(_LatAttnConfig), _I, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _P]
lib.ktx_latattn_mfma_eligible.argtypes = [C.POINTER(_LatAttnConfig)]
lib.ktx_latattn_mfma.argtypes = [C.POINTER(_LatAttnConfig), _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _P]
lib.ktx_moe_route.argtypes = [_I, _I, _I, _F, _F, _P, _L, _P, _P, _P]
lib.ktx_moe_plan.argtypes = [_I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P]
lib.ktx_grouped_gemv.argtypes = [_I, _I, _I, _P, _I, _L, _P, _P, _I, _P, _I, _L, _P, _I, _I, _P]
lib.ktx_grouped_gemm.argtypes = [_I, _I, _I, _I, _P, _I, _L, _L, _P, _P, _I, _P, _I, _L, _L, _P, _P, _P, _P, _I, _I, _I, _P]

TILE_M = 64
TILE_M_WIDE, WIDE_MIN_ROWS_PER_EXPERT = 128, 96      # bf16 steps whose experts average this many rows take 128-row tiles


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _f32(t, what):
    return None if t is None else _seq_dev(t, torch.float32, what)


def _i32(t, what):
    return None if t is None else _seq_dev(t, torch.int32, what)


def _rows_f32(t, what):
    """fp32 rows with unit inner stride (a column slice of a GEMM's output is fine) -> (pointer, row stride)."""
    if t is None:
        return None, 0
    if not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1:
        raise KtxError(f"{what}: expected fp32 rows on a HIP device, got {t.dtype} {tuple(t.shape)} strides {t.stride()}")
    return t.data_ptr(), t.stride(0)


def rows_add(x: torch.Tensor, x0: torch.Tensor | None = None, vec: torch.Tensor | None = None) -> torch.Tensor:
    """x[t] += x0[t] + vec, in place (ktx_rows_add)."""
    _f32(x, "rows_add x"), _f32(x0, "rows_add x0"), _f32(vec, "rows_add vec")
    T, W = x.shape
    if (x0 is not None and x0.shape != x.shape) or (vec is not None and vec.numel() != W):
        raise KtxError("rows_add: shapes do not fit")
    check(lib.ktx_rows_add(T, W, x.data_ptr(), _ptr(x0), _ptr(vec), _stream_ptr(x.device)))
    return x


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None, eps: float, rows: torch.Tensor | None = None,
               out_dtype=torch.float32) -> torch.Tensor:
    _f32(x, "layer_norm x"), _f32(w, "layer_norm w"), _f32(b, "layer_norm b"), _i32(rows, "layer_norm rows")
    W = x.shape[-1]
    T = rows.numel() if rows is not None else x.numel() // W
    if w.numel() != W or (b is not None and b.numel() != W):
        raise KtxError("layer_norm: weight / bias do not fit the row")
    out = torch.empty((T, W), dtype=out_dtype, device=x.device)
    check(lib.ktx_layer_norm(T, W, x.data_ptr(), w.data_ptr(), _ptr(b), float(eps), _ptr(rows), out.data_ptr(), SEQ_DTYPE[out_dtype],
                             _stream_ptr(x.device)))
    return out


def gated_norm_add(x: torch.Tensor, wn: torch.Tensor, bn: torch.Tensor | None, eps: float, y: torch.Tensor | None = None,
                   ybias: torch.Tensor | None = None, gate_logits: torch.Tensor | None = None, gate_bias: torch.Tensor | None = None,
                   expert_rows: torch.Tensor | None = None, pair_pos: torch.Tensor | None = None, topk_w: torch.Tensor | None = None,
                   next_norm: tuple | None = None):
    """x += layer_norm((y + ybias + sum_k topk_w[t, k] expert_rows[pair_pos[t, k]]) * sigmoid(gate_logits + gate_bias)), in place.
    next_norm = (weight, bias or None, eps, dtype): also returns layer_norm(updated x) in that type — (x, h) instead of x."""
    _f32(x, "gated_norm_add x"), _f32(wn, "wn"), _f32(bn, "bn"), _f32(ybias, "ybias"), _f32(gate_bias, "gate_bias")
    _f32(expert_rows, "expert_rows"), _i32(pair_pos, "pair_pos"), _f32(topk_w, "topk_w")
    T, W = x.shape
    yp, ldy = _rows_f32(y, "gated_norm_add y")
    gp, ldg = _rows_f32(gate_logits, "gated_norm_add gate_logits")
    for t in (y, gate_logits):
        if t is not None and tuple(t.shape) != (T, W):
            raise KtxError("gated_norm_add: y / gate_logits must be [T, W]")
    top = 0
    if expert_rows is not None:
        top = topk_w.shape[1]
        if expert_rows.shape[1] != W or pair_pos.numel() != T * top or topk_w.shape[0] != T:
            raise KtxError("gated_norm_add: the gathered term does not fit")
    h, nw, nb, neps, ndt = None, None, None, 0.0, torch.float32
    if next_norm is not None:
        nw, nb, neps, ndt = next_norm
        _f32(nw, "gated_norm_add next weight"), _f32(nb, "gated_norm_add next bias")
        if nw.numel() != W or (nb is not None and nb.numel() != W):
            raise KtxError("gated_norm_add: the following norm does not fit the row")
        h = torch.empty((T, W), dtype=ndt, device=x.device)
    check(lib.ktx_gated_norm_add(T, W, yp, ldy, _ptr(ybias), _ptr(expert_rows), _ptr(pair_pos), _ptr(topk_w), top, gp, ldg, _ptr(gate_bias),
                                 wn.data_ptr(), _ptr(bn), float(eps), x.data_ptr(), _ptr(nw), _ptr(nb), float(neps), _ptr(h),
                                 SEQ_DTYPE[ndt], _stream_ptr(x.device)))
    return x if next_norm is None else (x, h)


def poly_norm(z: torch.Tensor, bias: torch.Tensor | None, coef: torch.Tensor, eps: float, out_dtype=torch.float32) -> torch.Tensor:
    zp, ldz = _rows_f32(z, "poly_norm z")
    _f32(bias, "poly_norm bias"), _f32(coef, "poly_norm coef")
    T, F = z.shape
    if coef.numel() != 4 or (bias is not None and bias.numel() != F):
        raise KtxError("poly_norm: four coefficients, a bias per entry")
    out = torch.empty((T, F), dtype=out_dtype, device=z.device)
    check(lib.ktx_poly_norm(T, F, zp, ldz, _ptr(bias), coef.data_ptr(), float(eps), out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(z.device)))
    return out


def silu_mul_rows(gu: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """[R, 2F] (gate | up) -> silu(gate) * up, [R, F]."""
    p, ld = _rows_f32(gu, "silu_mul_rows")
    R, F = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((R, F), dtype=out_dtype, device=gu.device)
    check(lib.ktx_silu_mul_rows(R, F, p, ld, out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(gu.device)))
    return out


def postnorm_mix(x_in: torch.Tensor, x_out: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None, eps: float, alpha: float = 1.0,
                 y: torch.Tensor | None = None, ybias: torch.Tensor | None = None, stack: torch.Tensor | None = None, level: int = 0,
                 dwa: torch.Tensor | None = None, lp_dtype=None):
    """One launch (ktx_postnorm_mix): v = layer_norm(alpha * x_in + y + ybias; w, b, eps); with stack fp32 [levels, T, W], level `level`
    receives v, and with dwa fp32 [level + 1] the rows handed on are sum_j dwa[j] * stack[j]; x_out fp32 [T, W] (may be x_in) receives
    them.  Returns a copy of x_out in lp_dtype when that is given (what the following products read), else x_out."""
    _f32(x_in, "postnorm_mix x_in"), _f32(x_out, "postnorm_mix x_out"), _f32(w, "postnorm_mix w"), _f32(b, "postnorm_mix b")
    _f32(ybias, "postnorm_mix ybias"), _f32(stack, "postnorm_mix stack"), _f32(dwa, "postnorm_mix dwa")
    T, W = x_in.shape
    yp, ldy = _rows_f32(y, "postnorm_mix y")
    if tuple(x_out.shape) != (T, W) or w.numel() != W or (b is not None and b.numel() != W) or (ybias is not None and ybias.numel() != W) or \
            (y is not None and tuple(y.shape) != (T, W)):
        raise KtxError("postnorm_mix: shapes do not fit")
    if stack is not None and (stack.dim() != 3 or tuple(stack.shape[1:]) != (T, W) or not 0 <= level < stack.shape[0]):
        raise KtxError("postnorm_mix: stack must be [levels, T, W] with level inside")
    if dwa is not None and (stack is None or dwa.numel() != level + 1):
        raise KtxError("postnorm_mix: the average takes level + 1 weights and the stack")
    lp = torch.empty((T, W), dtype=lp_dtype, device=x_in.device) if lp_dtype is not None and lp_dtype != torch.float32 else None
    a = _PostNormArgs(yp, ldy, _ptr(ybias), float(alpha), w.data_ptr(), _ptr(b), float(eps), _ptr(stack),
                      stack.stride(0) if stack is not None else 0, int(level), _ptr(dwa), _ptr(lp), SEQ_DTYPE[lp.dtype] if lp is not None else 0)
    check(lib.ktx_postnorm_mix(T, W, x_in.data_ptr(), x_out.data_ptr(), C.byref(a), _stream_ptr(x_in.device)))
    return x_out if lp is None else lp


def glu_clamp_rows(gu: torch.Tensor, limit: float | None, slope: float = 1.0, up_shift: float = 0.0, out_dtype=torch.float32,
                   paired: bool = False) -> torch.Tensor:
    """[R, 2F] (gate | up; paired: gate_0, up_0, gate_1, up_1, ...) -> g * sigmoid(slope * g) * (u + up_shift), g = min(gate, limit),
    u = clamp(up, -limit, limit); [R, F] (ktx_glu_clamp_rows; limit None: neither is bounded)."""
    p, ld = _rows_f32(gu, "glu_clamp_rows")
    R, F = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((R, F), dtype=out_dtype, device=gu.device)
    check(lib.ktx_glu_clamp_rows(R, F, p, ld, float("inf") if limit is None else float(limit), float(slope), float(up_shift),
                                 1 if paired else 0, out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(gu.device)))
    return out


def sigmoid_gate_rows(o: torch.Tensor, gate: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """o [R, N] (contiguous, fp32 | bf16) * sigmoid(gate), gate fp32 rows [R, N] (a column slice is fine) -> [R, N] of out_dtype."""
    gp, ldg = _rows_f32(gate, "sigmoid_gate_rows gate")
    if o.dim() != 2 or not o.is_contiguous() or o.dtype not in SEQ_DTYPE or tuple(gate.shape) != tuple(o.shape):
        raise KtxError("sigmoid_gate_rows: o must be contiguous rows of the gate's shape")
    out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
    check(lib.ktx_sigmoid_gate_rows(o.shape[0], o.shape[1], o.data_ptr(), SEQ_DTYPE[o.dtype], gp, ldg, out.data_ptr(), SEQ_DTYPE[out_dtype],
                                    _stream_ptr(o.device)))
    return out


def head_gate_norm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, heads: int, vdim: int, eps: float, w_per_head: bool, act: str,
                   out_dtype=torch.float32) -> torch.Tensor:
    _f32(o, "head_gate_norm o"), _f32(w, "head_gate_norm w")
    gp, ldg = _rows_f32(gate, "head_gate_norm gate")
    T = o.shape[0]
    if o.numel() != T * heads * vdim or gate.shape[1] != heads * vdim or w.numel() != (heads * vdim if w_per_head else vdim):
        raise KtxError("head_gate_norm: shapes do not fit")
    out = torch.empty((T, heads * vdim), dtype=out_dtype, device=o.device)
    check(lib.ktx_head_gate_norm(T, heads, vdim, float(eps), o.data_ptr(), gp, ldg, w.data_ptr(), int(w_per_head),
                                 {"sigmoid": 0, "silu": 1}[act], out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(o.device)))
    return out


def delta_config(heads: int, kv_heads: int, dim: int, vdim: int, taps: int, unit_eps: float) -> _DeltaConfig:
    return _DeltaConfig(heads, kv_heads, dim, vdim, int(taps), float(unit_eps))


def delta_prep(cfg: _DeltaConfig, proj: torch.Tensor, offs: dict, taps: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor,
               batch, conv_state: torch.Tensor | None):
    """-> (qkv fp32 [T, C], gb fp32 [T, 2 heads + kv_heads]); the slots' convolution state moves on (ktx_delta_prep)."""
    pp, ldp = _rows_f32(proj, "delta_prep proj")
    _f32(taps, "taps"), _f32(A_log, "A_log"), _f32(dt_bias, "dt_bias"), _f32(conv_state, "conv_state")
    T = proj.shape[0]
    Cn = 2 * cfg.kv_heads * cfg.dim + cfg.heads * cfg.vdim
    if tuple(taps.shape) != (Cn, cfg.taps) or A_log.numel() != cfg.heads or dt_bias.numel() != cfg.heads:
        raise KtxError("delta_prep: taps [C, taps], A_log / dt_bias [heads]")
    if conv_state is not None and tuple(conv_state.shape[1:]) != (max(cfg.taps - 1, 1), Cn):
        raise KtxError("delta_prep: conv_state must be [slots, taps - 1, C]")
    qkv = torch.empty((T, Cn), dtype=torch.float32, device=proj.device)
    gb = torch.empty((T, 2 * cfg.heads + cfg.kv_heads), dtype=torch.float32, device=proj.device)
    check(lib.ktx_delta_prep(C.byref(cfg), batch.B, T, batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(),
                             batch.tok_req.data_ptr(), pp, ldp, offs["q"], offs["k"], offs["v"], offs["b"], offs["a"], taps.data_ptr(),
                             A_log.data_ptr(), dt_bias.data_ptr(), _ptr(conv_state), qkv.data_ptr(), gb.data_ptr(), _stream_ptr(proj.device)))
    return qkv, gb


def delta_forward(cfg: _DeltaConfig, qkv: torch.Tensor, gb: torch.Tensor, batch, S: torch.Tensor) -> torch.Tensor:
    _f32(qkv, "delta_forward qkv"), _f32(gb, "delta_forward gb"), _f32(S, "delta_forward S")
    if tuple(S.shape[1:]) != (cfg.heads, cfg.dim, cfg.vdim):
        raise KtxError("delta_forward: S must be [slots, heads, dim, vdim]")
    T = qkv.shape[0]
    o = torch.empty((T, cfg.heads * cfg.vdim), dtype=torch.float32, device=qkv.device)
    check(lib.ktx_delta_forward(C.byref(cfg), batch.B, batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(),
                                qkv.data_ptr(), gb.data_ptr(), S.data_ptr(), o.data_ptr(), _stream_ptr(qkv.device)))
    return o


def latattn_config(heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, rot_dims: int, scale: float, window: int, eps: float,
                   page_size: int, cache_dtype, rot_half: bool = False) -> _LatAttnConfig:
    return _LatAttnConfig(heads, dim, rot_dim, vdim, kv_rank, int(rot_dims), float(scale), int(window), float(eps), int(page_size),
                          SEQ_DTYPE[cache_dtype], 1 if rot_half else 0)


def latattn_prep(cfg: _LatAttnConfig, proj: torch.Tensor, q_off: int, c_off: int, wn: torch.Tensor | None, inv_freq: torch.Tensor,
                 positions: torch.Tensor, cache_loc: torch.Tensor, cache: torch.Tensor | None, q_out: torch.Tensor) -> None:
    """cache None (and wn None, c_off ignored): only the queries' rotated parts are written — the layer reads latent rows that another
    layer appended."""
    pp, ldp = _rows_f32(proj, "latattn_prep proj")
    _f32(wn, "latattn_prep wn"), _f32(q_out, "latattn_prep q_out"), _i32(positions, "positions"), _i32(cache_loc, "cache_loc")
    _seq_dev(inv_freq, torch.float64, "latattn_prep inv_freq")
    T, E = proj.shape[0], cfg.kv_rank + cfg.rot_dim
    if positions.numel() != T or cache_loc.numel() != T or q_out.numel() != T * cfg.heads * E or inv_freq.numel() != cfg.rot_dims // 2 or \
            proj.shape[1] < q_off + cfg.heads * (cfg.dim + cfg.rot_dim):
        raise KtxError("latattn_prep: shapes do not fit")
    if cache is not None and (cache.shape[-1] != E or wn is None or wn.numel() != cfg.kv_rank or not cache.is_contiguous()
                              or proj.shape[1] < c_off + E or int(cache.numel()) // E <= 0):
        raise KtxError("latattn_prep: cache / latent norm do not fit")
    check(lib.ktx_latattn_prep(C.byref(cfg), T, pp, ldp, q_off, c_off, _ptr(wn), inv_freq.data_ptr(), positions.data_ptr(),
                               cache_loc.data_ptr(), _ptr(cache), q_out.data_ptr(), _stream_ptr(proj.device)))


def latattn_forward(cfg: _LatAttnConfig, q: torch.Tensor, cache: torch.Tensor, batch, sink: torch.Tensor, nsplit: int = 1,
                    out_dtype=torch.float32) -> torch.Tensor:
    """-> [T, heads * kv_rank] of out_dtype: each head's softmax-weighted sum of latent rows (ktx_latattn_forward)."""
    _f32(q, "latattn_forward q"), _f32(sink, "latattn_forward sink")
    T, L = q.shape[0], cfg.kv_rank
    out = torch.empty((T, cfg.heads * L), dtype=out_dtype, device=q.device)
    scratch = torch.empty((nsplit, T, cfg.heads, L + 2), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_latattn_forward(C.byref(cfg), T, q.data_ptr(), cache.data_ptr(), batch.tok_req.data_ptr(), batch.positions.data_ptr(),
                                  batch.page_indptr.data_ptr(), batch.page_indices.data_ptr(), _ptr(sink), int(nsplit), _ptr(scratch),
                                  out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(q.device)))
    return out


def latattn_mfma_eligible(cfg: _LatAttnConfig) -> bool:
    return bool(lib.ktx_latattn_mfma_eligible(C.byref(cfg)))


def latattn_mfma(cfg: _LatAttnConfig, q: torch.Tensor, cache: torch.Tensor, batch, sink: torch.Tensor, nsplit: int = 1,
                 out_dtype=torch.bfloat16) -> torch.Tensor:
    """The matrix-core kernel, prompts and decode steps (ktx_latattn_mfma) -> [T, heads * kv_rank] of out_dtype."""
    _f32(q, "latattn_mfma q"), _f32(sink, "latattn_mfma sink")
    T, L = q.shape[0], cfg.kv_rank
    out = torch.empty((T, cfg.heads * L), dtype=out_dtype, device=q.device)
    scratch = torch.empty((nsplit, T, cfg.heads, L + 2), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_latattn_mfma(C.byref(cfg), batch.B, T, int(batch.max_q_len), q.data_ptr(), cache.data_ptr(), batch.q_indptr.data_ptr(),
                               batch.pos0.data_ptr(), batch.page_indptr.data_ptr(), batch.page_indices.data_ptr(), _ptr(sink),
                               int(nsplit), _ptr(scratch), out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(q.device)))
    return out


def moe_route(logits: torch.Tensor, top: int, scale: float, sum_eps: float):
    """logits fp32 rows [T, E] -> (topk_idx int32 [T, top], topk_w fp32 [T, top]) (ktx_moe_route)."""
    lp, ldl = _rows_f32(logits, "moe_route logits")
    T, E = logits.shape
    idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    check(lib.ktx_moe_route(T, E, top, float(scale), float(sum_eps), lp, ldl, idx.data_ptr(), w.data_ptr(), _stream_ptr(logits.device)))
    return idx, w


class MoePlan:
    __slots__ = ("group_off", "sorted_tok", "pair_pos", "sorted_group", "tile_group", "tile_row0", "num_tiles", "max_tiles", "pairs", "tile_m")


def moe_plan(topk_idx: torch.Tensor, E: int, wide: bool = False) -> MoePlan:
    """Sort the pairs by expert and lay the row tiles out (ktx_moe_plan).  wide: 128-row tiles (bf16 products of prompt-sized steps)."""
    _i32(topk_idx, "moe_plan topk_idx")
    T, top = topk_idx.shape
    p = MoePlan()
    p.pairs = T * top
    p.tile_m = TILE_M_WIDE if wide else TILE_M
    p.max_tiles = p.pairs // p.tile_m + min(E, p.pairs) + 1
    meta = torch.empty(E + 1 + 3 * p.pairs + 2 * p.max_tiles + 1, dtype=torch.int32, device=topk_idx.device)
    at = 0
    for name, n in (("group_off", E + 1), ("sorted_tok", p.pairs), ("pair_pos", p.pairs), ("sorted_group", p.pairs), ("tile_group", p.max_tiles),
                    ("tile_row0", p.max_tiles), ("num_tiles", 1)):
        setattr(p, name, meta[at:at + n])
        at += n
    check(lib.ktx_moe_plan(T, E, top, p.tile_m, topk_idx.data_ptr(), p.group_off.data_ptr(), p.sorted_tok.data_ptr(), p.pair_pos.data_ptr(),
                           p.sorted_group.data_ptr(), p.tile_group.data_ptr(), p.tile_row0.data_ptr(), p.num_tiles.data_ptr(), _stream_ptr(topk_idx.device)))
    return p


def _gg_types(a, w, out_dtype):
    if a.dtype not in SEQ_DTYPE or w.dtype not in SEQ_DTYPE or not a.is_cuda or a.stride(-1) != 1 or not w.is_contiguous():
        raise KtxError(f"grouped_gemm: {a.dtype} {tuple(a.shape)} x {w.dtype} {tuple(w.shape)} does not fit")
    if w.dtype == torch.float32 and (a.dtype != torch.float32 or out_dtype != torch.float32):
        raise KtxError("grouped_gemm: an fp32 product takes and writes fp32")


def head_gemm(a: torch.Tensor, a_goff: int, w: torch.Tensor, out: torch.Tensor, y_goff: int) -> torch.Tensor:
    """Per-head products: for g < G, out[:, g * y_goff : g * y_goff + N] = a[:, g * a_goff : g * a_goff + K] @ w[g]^T
    (w [G, N, K]; a, out 2-D rows whose columns may start anywhere — pass the views)."""
    G, N, K = w.shape
    _gg_types(a, w, out.dtype)
    M = a.shape[0]
    check(lib.ktx_grouped_gemm(G, M, N, K, a.data_ptr(), SEQ_DTYPE[a.dtype], a.stride(0), a_goff, None, w.data_ptr(), SEQ_DTYPE[w.dtype],
                               out.data_ptr(), SEQ_DTYPE[out.dtype], out.stride(0), y_goff, None, None, None, None, 0, TILE_M, 0, _stream_ptr(a.device)))
    return out


GEMV_MAX_ROWS = 64      # up to this many (token, choice) pairs a step's expert products stream the weights per row instead of tiling


GG_ACT = {None: 0, "none": 0, "glu_silu": 1, "relu_sq": 2}


def expert_gemm(a: torch.Tensor, w: torch.Tensor, plan: MoePlan, gather: bool, out_dtype=torch.float32, glu: bool = False,
                act: str | None = None) -> torch.Tensor:
    """Sorted row r (expert g = the group it falls in) : out[r] = a[plan.sorted_tok[r] if gather else r] @ w[g]^T.  w [E, N, K]; rows
    of groups >= E (a plan over more groups than there are weights) are left as they are.
    glu (only for steps of at most GEMV_MAX_ROWS pairs): w[g] = [gate ; up] and out[r] = silu(gate a) * (up a), [pairs, N / 2].
    act = "relu_sq": out = relu(out)^2 in the product's epilogue."""
    G, N, K = w.shape
    _gg_types(a, w, out_dtype)
    if glu and act:
        raise KtxError("expert_gemm: one epilogue")
    if plan.pairs <= GEMV_MAX_ROWS:
        n_out = N // 2 if glu else N
        out = torch.empty((plan.pairs, n_out), dtype=out_dtype, device=a.device)
        check(lib.ktx_grouped_gemv(plan.pairs, n_out, K, a.data_ptr(), SEQ_DTYPE[a.dtype], a.stride(0),
                                   plan.sorted_tok.data_ptr() if gather else None, w.data_ptr(), SEQ_DTYPE[w.dtype], out.data_ptr(),
                                   SEQ_DTYPE[out_dtype], out.stride(0), plan.sorted_group.data_ptr(), 1 if glu else GG_ACT[act], G,
                                   _stream_ptr(a.device)))
        return out
    if glu:
        raise KtxError("expert_gemm: the fused activation is the streaming form's (at most GEMV_MAX_ROWS pairs)")
    out = torch.empty((plan.pairs, N), dtype=out_dtype, device=a.device)
    check(lib.ktx_grouped_gemm(G, plan.pairs, N, K, a.data_ptr(), SEQ_DTYPE[a.dtype], a.stride(0), 0,
                               plan.sorted_tok.data_ptr() if gather else None, w.data_ptr(), SEQ_DTYPE[w.dtype], out.data_ptr(),
                               SEQ_DTYPE[out_dtype], out.stride(0), 0, plan.group_off.data_ptr(), plan.tile_group.data_ptr(),
                               plan.tile_row0.data_ptr(), plan.num_tiles.data_ptr(), plan.max_tiles, plan.tile_m, GG_ACT[act], _stream_ptr(a.device)))
    return out
