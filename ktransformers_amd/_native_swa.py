"""ctypes binding of include/ktx_swa.h — the residual update with a scalar-weight RMS norm, the input convolution over time,
grouped-query sliding-window attention over paged key and value caches (rotated values, a sink), the selective scan and the softmax
router.  Same library and calling rules as ktransformers_amd._native_seq: device pointers and the caller's current HIP stream cross the
boundary, every call is graph-capturable, there is no CPU fallback."""
from __future__ import annotations

import ctypes as C

import torch

from ktransformers_amd._native_seq import SEQ_DTYPE, KtxError, _seq_dev, _stream_ptr, check, lib

_P, _I, _L, _F, _I32 = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_int32


class _ResidArgs(C.Structure):       # include/ktx_swa.h: ktx_resid_args
    _fields_ = [("y", _P), ("ldy", _L), ("y_norm_w", _P), ("y_norm_eps", _F), ("ey", _P), ("pair_pos", _P), ("topk_idx", _P), ("topk_w", _P),
                ("top", _I32), ("n_real", _I32), ("h_in", _P), ("h_dtype", _I32), ("norm_g", _P), ("eps", _F), ("rows", _P), ("halo", _I32),
                ("B", _I32), ("q_indptr", _P), ("pos0", _P), ("slot", _P), ("tok_req", _P), ("conv_state", _P), ("conv_w", _P),
                ("conv_taps", _I32), ("out", _P), ("out_dtype", _I32)]


class _SwaConfig(C.Structure):       # include/ktx_swa.h: ktx_swa_config
    _fields_ = [("heads", _I32), ("kv_heads", _I32), ("dim", _I32), ("vdim", _I32), ("rot_dims", _I32), ("rot_values", _I32),
                ("qk_norm", _I32), ("eps", _F), ("scale", _F), ("window", _I32), ("page_size", _I32), ("cache_dtype", _I32),
                ("keep_first", _I32), ("bias_span", _I32)]


class _SsmConfig(C.Structure):       # include/ktx_swa.h: ktx_ssm_config
    _fields_ = [("inner", _I32), ("state", _I32), ("dt_rank", _I32), ("taps", _I32)]


if not hasattr(lib, "ktx_swa_forward"):
    raise ImportError("the loaded kernel library predates include/ktx_swa.h: rebuild with `python -m ktransformers_amd.build [--seq]`")
lib.ktx_resid_norm.argtypes = [_I, _I, _P, C.POINTER(_ResidArgs), _P]
lib.ktx_input_conv.argtypes = [_I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P]
lib.ktx_rows_mul_lookup.argtypes = [_I, _I, _P, _L, _P, _I, _L, _I, _P, _P, _I, _P]
lib.ktx_swa_prep.argtypes = [C.POINTER(_SwaConfig), _I, _P, _L, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P]
lib.ktx_swa_conv_prep.argtypes = [C.POINTER(_SwaConfig), _I, _I, _I, _I, _P, _L] + [_P] * 14
lib.ktx_swa_forward.argtypes = [C.POINTER(_SwaConfig), _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _P]
lib.ktx_swa_mfma_eligible.argtypes = [C.POINTER(_SwaConfig)]
lib.ktx_swa_mfma.argtypes = [C.POINTER(_SwaConfig), _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I, _P]
lib.ktx_ssm_conv.argtypes = [C.POINTER(_SsmConfig), _I, _I, _P, _P, _P, _P, _P, _L, _I, _P, _P, _P, _P, _P]
lib.ktx_ssm_scan.argtypes = [C.POINTER(_SsmConfig), _I, _I, _I, _P, _P, _P, _P, _P, _P, _L, _P, _L, _P, _P, _P, _P, _L, _I, _I, _P, _P, _P,
                             _I, _P]
lib.ktx_softmax_route.argtypes = [_I, _I, _I, _F, _P, _L, _P, _P, _P, _P]
lib.ktx_softmax_route_plan.argtypes = [_I, _I, _I, _F, _P, _L, _P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P]


FUSED_CONV_MAX_TAPS = 9      # ktx_resid_norm's one-token form keeps the state rows of one channel in registers


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


def resid_norm(x: torch.Tensor, y: torch.Tensor | None = None, y_norm: tuple | None = None, moe: tuple | None = None,
               norm: tuple | None = None, halo: tuple | None = None, rows: torch.Tensor | None = None, out_dtype=torch.float32,
               conv: tuple | None = None):
    """One launch (ktx_resid_norm): x [T, W] fp32 += y (with y_norm = (weight [W], eps): y / rms(y) * weight first)
    + the mixture's weighted sum, moe = (expert_rows [pairs, W], pair_pos, topk_idx, topk_w [T, top], n_real, h_in [T, W]); then, with
    norm = (g: one fp32 number on the device, eps), returns x * g / rms(x) — in out_dtype [T or len(rows), W], or, with
    halo = (taps - 1, batch, conv_state [slots, taps - 1, W]), as fp32 [T + B * halo, W] with every request's state rows in front of
    its tokens (what input_conv reads).  conv = (taps weight fp32 [W, taps], batch, conv_state), for steps in which every request brings
    exactly ONE token: h + conv(h) in out_dtype [T, W] from the same launch, the slots' state moved on (a one-tap convolution has no
    state and takes any step)."""
    _f32(x, "resid_norm x")
    T, W = x.shape
    a = _ResidArgs()
    if y is not None:
        a.y, a.ldy = _rows_f32(y, "resid_norm y")
        if tuple(y.shape) != (T, W):
            raise KtxError("resid_norm: y must be [T, W]")
        if y_norm is not None:
            w, eps = y_norm
            _f32(w, "resid_norm y_norm weight")
            if w.numel() != W:
                raise KtxError("resid_norm: y_norm weight must be [W]")
            a.y_norm_w, a.y_norm_eps = w.data_ptr(), float(eps)
    if moe is not None:
        ey, pair_pos, topk_idx, topk_w, n_real, h_in = moe
        _f32(ey, "resid_norm expert rows"), _i32(pair_pos, "pair_pos"), _i32(topk_idx, "topk_idx"), _f32(topk_w, "topk_w")
        _seq_dev(h_in, None, "resid_norm h_in")
        top = topk_w.shape[1]
        if ey.shape[1] != W or pair_pos.numel() != T * top or tuple(topk_idx.shape) != (T, top) or topk_w.shape[0] != T or \
                tuple(h_in.shape) != (T, W) or h_in.dtype not in SEQ_DTYPE:
            raise KtxError("resid_norm: the mixture's term does not fit")
        a.ey, a.pair_pos, a.topk_idx, a.topk_w = ey.data_ptr(), pair_pos.data_ptr(), topk_idx.data_ptr(), topk_w.data_ptr()
        a.top, a.n_real, a.h_in, a.h_dtype = top, int(n_real), h_in.data_ptr(), SEQ_DTYPE[h_in.dtype]
    out = None
    if norm is not None:
        g, eps = norm
        _f32(g, "resid_norm g")
        a.norm_g, a.eps = g.data_ptr(), float(eps)
        n_out = T
        if rows is not None:
            _i32(rows, "resid_norm rows")
            a.rows, n_out = rows.data_ptr(), rows.numel()
        if halo is not None:
            h, batch, state = halo
            _f32(state, "resid_norm conv_state")
            if tuple(state.shape[1:]) != (h, W) or out_dtype != torch.float32:
                raise KtxError("resid_norm: conv_state must be [slots, halo, W] and the rows fp32")
            a.halo, a.B = int(h), int(batch.B)
            a.q_indptr, a.pos0, a.slot, a.tok_req = (batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(),
                                                     batch.tok_req.data_ptr())
            a.conv_state = state.data_ptr()
            n_out = T + batch.B * h
        if conv is not None:
            cw, batch, state = conv
            _f32(cw, "resid_norm conv weight"), _f32(state, "resid_norm conv_state")
            taps = cw.shape[1]
            if halo is not None or rows is not None or cw.shape[0] != W or not 1 <= taps <= FUSED_CONV_MAX_TAPS:
                raise KtxError("resid_norm: the fused convolution takes 1 .. 9 taps [W, taps], no halo, no row gather")
            a.conv_w, a.conv_taps = cw.data_ptr(), taps
            if taps > 1:
                if batch.max_q_len != 1 or batch.T != T or state is None or tuple(state.shape[1:]) != (taps - 1, W):
                    raise KtxError("resid_norm: beyond one tap the fused convolution takes one token per request and a state [slots, taps - 1, W]")
                a.B = int(batch.B)
                a.q_indptr, a.pos0, a.slot, a.tok_req = (batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(),
                                                         batch.tok_req.data_ptr())
                a.conv_state = state.data_ptr()
        out = torch.empty((n_out, W), dtype=out_dtype, device=x.device)
        a.out, a.out_dtype = out.data_ptr(), SEQ_DTYPE[out_dtype]
    check(lib.ktx_resid_norm(rows.numel() if rows is not None else T, W, x.data_ptr(), C.byref(a), _stream_ptr(x.device)))
    return out


def input_conv(hx: torch.Tensor, w: torch.Tensor, batch, conv_state: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """hx fp32 [T + B * (taps - 1), W] as resid_norm lays it out; w fp32 [W, taps] -> h + conv(h), [T, W] of out_dtype; the slots'
    state moves on (ktx_input_conv)."""
    _f32(hx, "input_conv hx"), _f32(w, "input_conv w"), _f32(conv_state, "input_conv state")
    W, taps = w.shape
    T = hx.shape[0] - batch.B * (taps - 1)
    if hx.shape[1] != W or T != batch.T or tuple(conv_state.shape[1:]) != (taps - 1, W):
        raise KtxError("input_conv: shapes do not fit")
    out = torch.empty((T, W), dtype=out_dtype, device=hx.device)
    check(lib.ktx_input_conv(batch.B, T, W, taps, hx.data_ptr(), w.data_ptr(), batch.q_indptr.data_ptr(), batch.slot.data_ptr(),
                             batch.tok_req.data_ptr(), conv_state.data_ptr(), out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(hx.device)))
    return out


def rows_mul_lookup(a: torch.Tensor, table: torch.Tensor, col0: int, tokens: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """a fp32 rows [T, n] times table[tokens][:, col0 : col0 + n] -> [T, n] of out_dtype (ktx_rows_mul_lookup)."""
    ap, lda = _rows_f32(a, "rows_mul_lookup a")
    _i32(tokens, "rows_mul_lookup tokens")
    T, n = a.shape
    if table.dim() != 2 or table.stride(1) != 1 or table.dtype not in SEQ_DTYPE or col0 + n > table.shape[1] or tokens.numel() != T:
        raise KtxError("rows_mul_lookup: shapes do not fit")
    out = torch.empty((T, n), dtype=out_dtype, device=a.device)
    check(lib.ktx_rows_mul_lookup(T, n, ap, lda, table.data_ptr(), SEQ_DTYPE[table.dtype], table.stride(0), int(col0), tokens.data_ptr(),
                                  out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(a.device)))
    return out


def swa_config(heads: int, kv_heads: int, dim: int, vdim: int, rot_dims: int, rot_values: bool, qk_norm: bool, eps: float, scale: float,
               window: int, page_size: int, cache_dtype, keep_first: int = 0, bias_span: int = 0) -> _SwaConfig:
    """keep_first: with a window, the sequence's first positions that stay visible; bias_span: rows - 1 of the distance-bias table the
    attention calls are given (`dist_bias`)."""
    return _SwaConfig(heads, kv_heads, dim, vdim, int(rot_dims), int(bool(rot_values)), int(bool(qk_norm)), float(eps), float(scale),
                      int(window), int(page_size), SEQ_DTYPE[cache_dtype], int(keep_first), int(bias_span))


def swa_conv_prep(cfg: _SwaConfig, proj: torch.Tensor, bias: torch.Tensor | None, conv_w: torch.Tensor | None, q_norm_w: torch.Tensor | None,
                  k_norm_w: torch.Tensor | None, batch, conv_state: torch.Tensor | None, kcache: torch.Tensor, vcache: torch.Tensor) -> torch.Tensor:
    """The un-rotated prep with a causal convolution over time behind the projections and RMS norms over the whole q and k projections
    (ktx_swa_conv_prep): proj fp32 [T, >= C] with q | k | v at column 0 -> q fp32 [T, heads * dim] (normed, scaled); key and value rows
    are appended, the convolution's state slots move on.  conv_w fp32 [C, taps] or None."""
    pp, ldp = _rows_f32(proj, "swa_conv_prep proj")
    for t_, what in ((bias, "bias"), (conv_w, "conv_w"), (q_norm_w, "q_norm_w"), (k_norm_w, "k_norm_w"), (conv_state, "conv_state")):
        _f32(t_, "swa_conv_prep " + what)
    T = proj.shape[0]
    nq, nk, nv = cfg.heads * cfg.dim, cfg.kv_heads * cfg.dim, cfg.kv_heads * cfg.vdim
    Cn = nq + nk + nv
    taps = int(conv_w.shape[1]) if conv_w is not None else 0
    if batch.positions.numel() != T or batch.cache_loc.numel() != T or proj.shape[1] < Cn or \
            tuple(kcache.shape[1:]) != (cfg.kv_heads, cfg.dim) or tuple(vcache.shape[1:]) != (cfg.kv_heads, cfg.vdim) or \
            not kcache.is_contiguous() or not vcache.is_contiguous() or kcache.dtype != vcache.dtype or \
            SEQ_DTYPE.get(kcache.dtype) != cfg.cache_dtype or (bias is not None and bias.numel() != Cn) or \
            (conv_w is not None and tuple(conv_w.shape) != (Cn, taps)) or (q_norm_w is not None and q_norm_w.numel() != nq) or \
            (k_norm_w is not None and k_norm_w.numel() != nk) or \
            (taps > 1 and (conv_state is None or tuple(conv_state.shape[1:]) != (taps - 1, Cn))):
        raise KtxError("swa_conv_prep: shapes do not fit")
    q = torch.empty((T, nq), dtype=torch.float32, device=proj.device)
    check(lib.ktx_swa_conv_prep(C.byref(cfg), batch.B, T, int(batch.max_q_len), taps, pp, ldp, _ptr(bias), _ptr(conv_w), _ptr(q_norm_w), _ptr(k_norm_w),
                                batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(), batch.tok_req.data_ptr(),
                                _ptr(conv_state), batch.cache_loc.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), q.data_ptr(),
                                _stream_ptr(proj.device)))
    return q


def swa_prep(cfg: _SwaConfig, proj: torch.Tensor, q_off: int, k_off: int, v_off: int, inv_freq: torch.Tensor | None,
             v_inv_freq: torch.Tensor | None, positions: torch.Tensor, cache_loc: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor):
    """-> (q fp32 [T, heads * dim] rotated, normed, scaled; vcs fp32 [T, vdim] or None); the step's key and value rows are appended."""
    pp, ldp = _rows_f32(proj, "swa_prep proj")
    _i32(positions, "positions"), _i32(cache_loc, "cache_loc")
    T = proj.shape[0]
    if positions.numel() != T or cache_loc.numel() != T or tuple(kcache.shape[1:]) != (cfg.kv_heads, cfg.dim) or \
            tuple(vcache.shape[1:]) != (cfg.kv_heads, cfg.vdim) or not kcache.is_contiguous() or not vcache.is_contiguous() or \
            kcache.dtype != vcache.dtype or SEQ_DTYPE.get(kcache.dtype) != cfg.cache_dtype:
        raise KtxError("swa_prep: shapes do not fit")
    if cfg.rot_dims and (inv_freq is None or inv_freq.dtype != torch.float64 or inv_freq.numel() != cfg.rot_dims // 2):
        raise KtxError("swa_prep: inv_freq must be fp64 [rot_dims / 2]")
    if cfg.rot_values and (v_inv_freq is None or v_inv_freq.dtype != torch.float64 or v_inv_freq.numel() != cfg.vdim // 2):
        raise KtxError("swa_prep: v_inv_freq must be fp64 [vdim / 2]")
    q = torch.empty((T, cfg.heads * cfg.dim), dtype=torch.float32, device=proj.device)
    vcs = torch.empty((T, cfg.vdim), dtype=torch.float32, device=proj.device) if cfg.rot_values else None
    check(lib.ktx_swa_prep(C.byref(cfg), T, pp, ldp, q_off, k_off, v_off, _ptr(inv_freq) if cfg.rot_dims else None,
                           _ptr(v_inv_freq) if cfg.rot_values else None, positions.data_ptr(), cache_loc.data_ptr(), kcache.data_ptr(),
                           vcache.data_ptr(), q.data_ptr(), _ptr(vcs), _stream_ptr(proj.device)))
    return q, vcs


def _dist_bias_ok(cfg: _SwaConfig, dist_bias) -> None:
    _f32(dist_bias, "dist_bias")
    if dist_bias is not None and tuple(dist_bias.shape) != (cfg.bias_span + 1, cfg.heads):
        raise KtxError(f"dist_bias: expected fp32 [{cfg.bias_span + 1}, {cfg.heads}], got {tuple(dist_bias.shape)}")


def swa_forward(cfg: _SwaConfig, q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, batch, sink: torch.Tensor | None,
                vcs: torch.Tensor | None, nsplit: int = 1, out_dtype=torch.float32, dist_bias: torch.Tensor | None = None) -> torch.Tensor:
    """The vector-ALU form (ktx_swa_forward) -> [T, heads * vdim] of out_dtype.  dist_bias fp32 [cfg.bias_span + 1, heads]: added to the
    score by distance (the last row serves every larger distance)."""
    _f32(q, "swa_forward q"), _f32(sink, "swa_forward sink"), _f32(vcs, "swa_forward vcs"), _dist_bias_ok(cfg, dist_bias)
    T = q.shape[0]
    out = torch.empty((T, cfg.heads * cfg.vdim), dtype=out_dtype, device=q.device)
    scratch = torch.empty((nsplit, T, cfg.heads, cfg.vdim + 2), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_swa_forward(C.byref(cfg), T, q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), batch.tok_req.data_ptr(),
                              batch.positions.data_ptr(), batch.page_indptr.data_ptr(), batch.page_indices.data_ptr(), _ptr(sink),
                              _ptr(dist_bias), _ptr(vcs), int(nsplit), _ptr(scratch), out.data_ptr(), SEQ_DTYPE[out_dtype], _stream_ptr(q.device)))
    return out


def swa_mfma_eligible(cfg: _SwaConfig) -> bool:
    return bool(lib.ktx_swa_mfma_eligible(C.byref(cfg)))


def swa_mfma(cfg: _SwaConfig, q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, batch, sink: torch.Tensor | None,
             vcs: torch.Tensor | None, nsplit: int = 1, out_dtype=torch.bfloat16, dist_bias: torch.Tensor | None = None) -> torch.Tensor:
    """The matrix-core form, prompts and decode steps (ktx_swa_mfma) -> [T, heads * vdim] of out_dtype."""
    _f32(q, "swa_mfma q"), _f32(sink, "swa_mfma sink"), _f32(vcs, "swa_mfma vcs"), _dist_bias_ok(cfg, dist_bias)
    T = q.shape[0]
    out = torch.empty((T, cfg.heads * cfg.vdim), dtype=out_dtype, device=q.device)
    scratch = torch.empty((nsplit, T, cfg.heads, cfg.vdim + 2), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_swa_mfma(C.byref(cfg), batch.B, T, int(batch.max_q_len), q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(),
                           batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.page_indptr.data_ptr(), batch.page_indices.data_ptr(),
                           _ptr(sink), _ptr(dist_bias), _ptr(vcs), int(nsplit), _ptr(scratch), out.data_ptr(), SEQ_DTYPE[out_dtype],
                           _stream_ptr(q.device)))
    return out


def ssm_config(inner: int, state: int, dt_rank: int, taps: int) -> _SsmConfig:
    return _SsmConfig(int(inner), int(state), int(dt_rank), int(taps))


def ssm_conv(cfg: _SsmConfig, proj: torch.Tensor, x_off: int, w: torch.Tensor, bias: torch.Tensor | None, batch,
             conv_state: torch.Tensor | None) -> torch.Tensor:
    """-> silu(conv(x) + bias) fp32 [T, inner] (ktx_ssm_conv; the state is moved on by ssm_scan)."""
    pp, ldp = _rows_f32(proj, "ssm_conv proj")
    _f32(w, "ssm_conv w"), _f32(bias, "ssm_conv bias"), _f32(conv_state, "ssm_conv state")
    T = proj.shape[0]
    if tuple(w.shape) != (cfg.inner, cfg.taps) or (bias is not None and bias.numel() != cfg.inner) or \
            (cfg.taps > 1 and tuple(conv_state.shape[1:]) != (cfg.taps - 1, cfg.inner)):
        raise KtxError("ssm_conv: shapes do not fit")
    xc = torch.empty((T, cfg.inner), dtype=torch.float32, device=proj.device)
    check(lib.ktx_ssm_conv(C.byref(cfg), batch.B, T, batch.q_indptr.data_ptr(), batch.pos0.data_ptr(), batch.slot.data_ptr(),
                           batch.tok_req.data_ptr(), pp, ldp, int(x_off), w.data_ptr(), _ptr(bias), _ptr(conv_state), xc.data_ptr(),
                           _stream_ptr(proj.device)))
    return xc


def ssm_scan(cfg: _SsmConfig, xc: torch.Tensor, Bm: torch.Tensor, Cm: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor,
             A_log: torch.Tensor, D: torch.Tensor, proj: torch.Tensor, x_off: int, z_off: int, batch, S: torch.Tensor,
             conv_state: torch.Tensor | None, out_dtype=torch.float32) -> torch.Tensor:
    """The recurrence over the step's tokens (ktx_ssm_scan) -> y * silu(z), [T, inner] of out_dtype; S and the convolution's state move on."""
    _f32(xc, "ssm_scan xc"), _f32(dt_bias, "dt_bias"), _f32(A_log, "A_log"), _f32(D, "D"), _f32(S, "S"), _f32(conv_state, "conv state")
    bp, ldbc = _rows_f32(Bm, "ssm_scan B")
    cp, ldc = _rows_f32(Cm, "ssm_scan C")
    dp, lddt = _rows_f32(dt_raw, "ssm_scan dt")
    pp, ldp = _rows_f32(proj, "ssm_scan proj")
    T = xc.shape[0]
    if ldc != ldbc or Bm.shape[1] != cfg.state or Cm.shape[1] != cfg.state or tuple(dt_raw.shape) != (T, cfg.inner) or \
            tuple(A_log.shape) != (cfg.inner, cfg.state) or dt_bias.numel() != cfg.inner or D.numel() != cfg.inner or \
            tuple(S.shape[1:]) != (cfg.inner, cfg.state) or tuple(xc.shape) != (T, cfg.inner):
        raise KtxError("ssm_scan: shapes do not fit")
    out = torch.empty((T, cfg.inner), dtype=out_dtype, device=xc.device)
    check(lib.ktx_ssm_scan(C.byref(cfg), batch.B, T, int(batch.max_q_len), batch.q_indptr.data_ptr(), batch.pos0.data_ptr(),
                           batch.slot.data_ptr(), xc.data_ptr(), bp, cp, ldbc, dp, lddt, dt_bias.data_ptr(), A_log.data_ptr(), D.data_ptr(),
                           pp, ldp, int(x_off), int(z_off), S.data_ptr(), _ptr(conv_state), out.data_ptr(), SEQ_DTYPE[out_dtype],
                           _stream_ptr(xc.device)))
    return out


def softmax_route(logits: torch.Tensor, top: int, sum_eps: float, correction: torch.Tensor | None = None):
    """logits fp32 rows [T, E] -> (topk_idx int32 [T, top], topk_w fp32 [T, top]) (ktx_softmax_route)."""
    lp, ldl = _rows_f32(logits, "softmax_route logits")
    _f32(correction, "softmax_route correction")
    T, E = logits.shape
    if correction is not None and correction.numel() != E:
        raise KtxError("softmax_route: one correction per router output")
    idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    check(lib.ktx_softmax_route(T, E, top, float(sum_eps), lp, ldl, _ptr(correction), idx.data_ptr(), w.data_ptr(), _stream_ptr(logits.device)))
    return idx, w


ROUTE_PLAN_MAX_T = 64        # up to this many tokens a step routes and sorts in one launch (ktx_softmax_route_plan takes up to 256)


def softmax_route_plan(logits: torch.Tensor, top: int, sum_eps: float, correction: torch.Tensor | None = None):
    """softmax_route and the expert sort over all E router outputs (ktransformers_amd._native_hyb.moe_plan, 64-row tiles) in ONE launch,
    for small steps -> (topk_idx, topk_w, plan)."""
    from ktransformers_amd._native_hyb import TILE_M, MoePlan
    lp, ldl = _rows_f32(logits, "softmax_route_plan logits")
    _f32(correction, "softmax_route_plan correction")
    T, E = logits.shape
    if correction is not None and correction.numel() != E:
        raise KtxError("softmax_route_plan: one correction per router output")
    idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    p = MoePlan()
    p.pairs, p.tile_m = T * top, TILE_M
    p.max_tiles = p.pairs // p.tile_m + min(E, p.pairs) + 1
    meta = torch.empty(E + 1 + 3 * p.pairs + 2 * p.max_tiles + 1, dtype=torch.int32, device=logits.device)
    at = 0
    for name, n in (("group_off", E + 1), ("sorted_tok", p.pairs), ("pair_pos", p.pairs), ("sorted_group", p.pairs), ("tile_group", p.max_tiles),
                    ("tile_row0", p.max_tiles), ("num_tiles", 1)):
        setattr(p, name, meta[at:at + n])
        at += n
    check(lib.ktx_softmax_route_plan(T, E, top, float(sum_eps), lp, ldl, _ptr(correction), idx.data_ptr(), w.data_ptr(), p.tile_m,
                                     p.group_off.data_ptr(), p.sorted_tok.data_ptr(), p.pair_pos.data_ptr(), p.sorted_group.data_ptr(),
                                     p.tile_group.data_ptr(), p.tile_row0.data_ptr(), p.num_tiles.data_ptr(), _stream_ptr(logits.device)))
    return idx, w, p
