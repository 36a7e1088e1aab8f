"""ctypes binding of include/ktx_seq.h — the sequence-mixer kernels (sigmoid attention over a paged key cache, the mLSTM
recurrence over state slots, the fp32-residual norm glue, a dense GEMM of any shape in bf16 or fp32).

The entry points live in libktx_hip.so; a checkout that has only built `libktx_seq.so` (`python -m ktransformers_amd.build --seq`:
csrc/ktx_seq.hip + the error plumbing, seconds instead of minutes) serves models that need nothing else.  Device pointers and the
caller's current HIP stream cross the boundary, so every call is graph-capturable.  No CPU fallback: the import raises when
neither library exists."""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATHS = (os.path.join(_HERE, "lib", "libktx_hip.so"), os.path.join(_HERE, "lib", "libktx_seq.so"))


class KtxError(RuntimeError):
    pass


class _SigAttnConfig(C.Structure):   # include/ktx_seq.h: ktx_sigattn_config
    _fields_ = [("heads", C.c_int32), ("kv_heads", C.c_int32), ("dim", C.c_int32), ("scale", C.c_float), ("temp_coef", C.c_float),
                ("temp_every", C.c_int32), ("slope_span", C.c_float), ("page_size", C.c_int32), ("cache_dtype", C.c_int32)]


class _MlstmConfig(C.Structure):     # include/ktx_seq.h: ktx_mlstm_config
    _fields_ = [("heads", C.c_int32), ("dim", C.c_int32), ("vdim", C.c_int32), ("gate_cap", C.c_float), ("eps", C.c_float),
                ("denom_eps", C.c_float)]



def _load() -> C.CDLL:
    have = [p for p in LIB_PATHS if os.path.exists(p)]
    # the whole library when it is there — unless the subset library was built after it (sources changed and only the subset was rebuilt)
    path = max(have, key=os.path.getmtime) if len(have) == 2 and os.path.getmtime(have[1]) > os.path.getmtime(have[0]) else (have[0] if have else None)
    if path is None:
        raise ImportError(f"neither {LIB_PATHS[0]} nor {LIB_PATHS[1]} found: build with `python -m ktransformers_amd.build [--seq]` "
                          "(hipcc, gfx950).  ktransformers_amd has no CPU fallback.")
    lib = C.CDLL(path)
    lib.ktx_last_error.restype = C.c_char_p
    # include/ktx_seq.h
    lib.ktx_embed_sinpos.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.ktx_dense_gemm.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int64, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                   C.c_int64, C.c_int, C.c_int, C.c_void_p]
    if hasattr(lib, "ktx_dense_gemv_glu"):
        lib.ktx_dense_gemv_glu.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int64, C.c_void_p, C.c_void_p, C.c_int, C.c_int64,
                                           C.c_float, C.c_float, C.c_float, C.c_void_p]
    lib.ktx_sigattn_prep.argtypes = [C.POINTER(_SigAttnConfig), C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                     C.c_float] + [C.c_void_p] * 6
    lib.ktx_sigattn_forward.argtypes = [C.POINTER(_SigAttnConfig), C.c_int] + [C.c_void_p] * 9 + [C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                                                                                                 C.c_void_p]
    lib.ktx_sigattn_prefill_eligible.argtypes = [C.POINTER(_SigAttnConfig)]
    lib.ktx_sigattn_prefill.argtypes = [C.POINTER(_SigAttnConfig), C.c_int, C.c_int, C.c_int] + [C.c_void_p] * 9 + [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.ktx_gelu_tanh.argtypes = [C.c_size_t, C.c_void_p, C.c_int, C.c_void_p]
    lib.ktx_mlstm_forward.argtypes = [C.POINTER(_MlstmConfig), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64] + [
        C.c_int] * 5 + [C.c_void_p] * 7 + [C.c_int, C.c_void_p]
    lib.ktx_mlstm_gate_norm.argtypes = [C.POINTER(_MlstmConfig), C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p,
                                        C.c_void_p, C.c_int, C.c_void_p]
    lib.ktx_rms_combine.argtypes = [C.c_int, C.c_int] + [C.c_void_p] * 5 + [C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p,
                                                                          C.c_int, C.c_void_p]
    return lib


lib = _load()


def check(rc: int) -> None:
    if rc != 0:
        raise KtxError(lib.ktx_last_error().decode("utf-8", "replace"))


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


SEQ_DTYPE = {torch.float32: 0, torch.bfloat16: 1}
ACT = {None: 0, "none": 0, "gelu_tanh": 1}


def _seq_dev(t: torch.Tensor, dtype, what: str) -> torch.Tensor:
    if not t.is_cuda or (dtype is not None and t.dtype != dtype) or not t.is_contiguous():
        raise KtxError(f"{what}: expected a contiguous {dtype} tensor on a HIP device, got {t.dtype} {tuple(t.shape)} on {t.device}")
    return t


def embed_sinpos(tokens: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """tokens, positions int32 [T]; embed [vocab, width] bf16 | fp32; inv_freq fp64 [(width + 1) // 2] -> fp32 [T, width]."""
    _seq_dev(tokens, torch.int32, "embed_sinpos tokens"), _seq_dev(positions, torch.int32, "embed_sinpos positions")
    _seq_dev(inv_freq, torch.float64, "embed_sinpos inv_freq"), _seq_dev(embed, None, "embed_sinpos embed")
    T, (vocab, width) = tokens.numel(), embed.shape
    if positions.numel() != T or inv_freq.numel() != (width + 1) // 2 or embed.dtype not in SEQ_DTYPE:
        raise KtxError("embed_sinpos: shapes / element type do not fit")
    x = torch.empty((T, width), dtype=torch.float32, device=tokens.device)
    check(lib.ktx_embed_sinpos(T, width, vocab, tokens.data_ptr(), positions.data_ptr(), embed.data_ptr(), SEQ_DTYPE[embed.dtype],
                               inv_freq.data_ptr(), x.data_ptr(), _stream_ptr(x.device)))
    return x


def embed_rows(tokens: torch.Tensor, embed: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """tokens int32 [T]; embed [vocab, width] bf16 | fp32 -> the table rows as fp32 [T, width] (ktx_embed_sinpos without positions);
    `out`: a contiguous fp32 [T, width] tensor to write them into."""
    _seq_dev(tokens, torch.int32, "embed_rows tokens"), _seq_dev(embed, None, "embed_rows embed")
    if embed.dtype not in SEQ_DTYPE:
        raise KtxError("embed_rows: element type does not fit")
    T, (vocab, width) = tokens.numel(), embed.shape
    if out is not None and (tuple(_seq_dev(out, torch.float32, "embed_rows out").shape) != (T, width)):
        raise KtxError("embed_rows: out must be fp32 [T, width]")
    x = out if out is not None else torch.empty((T, width), dtype=torch.float32, device=tokens.device)
    check(lib.ktx_embed_sinpos(T, width, vocab, tokens.data_ptr(), None, embed.data_ptr(), SEQ_DTYPE[embed.dtype], None, x.data_ptr(),
                               _stream_ptr(x.device)))
    return x


def dense_gemm(a: torch.Tensor, w: torch.Tensor, out_dtype=torch.float32, act: str | None = None, out: torch.Tensor | None = None,
               ksplit: int = 1) -> torch.Tensor:
    """a [M, K] (fp32 | bf16, unit inner stride) x w [N, K]^T (contiguous bf16 | fp32: its type is the product's) -> [M, N] of
    out_dtype (ktx_dense_gemm: any shape)."""
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1] or a.stride(1) != 1 or not w.is_contiguous() or not a.is_cuda \
            or a.device != w.device or a.dtype not in SEQ_DTYPE or w.dtype not in SEQ_DTYPE:
        raise KtxError(f"dense_gemm: {a.dtype} {tuple(a.shape)} x {w.dtype} {tuple(w.shape)}^T does not fit")
    M, K = a.shape
    N = w.shape[0]
    if (out is None and ksplit == 1 and M >= LIBRARY_GEMM_MIN_M and w.dtype == torch.bfloat16 and K % 64 == 0 and N % 8 == 0
            and _library_gemm() is not None):
        # prompt-sized bf16 products go to the library's tuned MFMA GEMM (include/ktx_gemm.h); the activation has its own launch
        a16 = a if a.dtype == torch.bfloat16 else a.to(torch.bfloat16)
        y = _library_gemm()(a16 if a16.stride(0) % 8 == 0 else a16.contiguous(), w, out_f32=out_dtype == torch.float32)
        if ACT[act]:
            check(lib.ktx_gelu_tanh(y.numel(), y.data_ptr(), SEQ_DTYPE[y.dtype], _stream_ptr(y.device)))
        return y
    if out is None:
        out = (torch.zeros if ksplit > 1 else torch.empty)((M, N), dtype=out_dtype, device=a.device)
    elif out.dtype != out_dtype or tuple(out.shape) != (M, N) or out.stride(1) != 1:
        raise KtxError("dense_gemm: out does not fit")
    check(lib.ktx_dense_gemm(M, N, K, a.data_ptr(), SEQ_DTYPE[a.dtype], a.stride(0), w.data_ptr(), SEQ_DTYPE[w.dtype], out.data_ptr(),
                             SEQ_DTYPE[out_dtype], out.stride(0), ACT[act], int(ksplit), _stream_ptr(a.device)))
    return out


GEMV_GLU_MAX_M = 16


def dense_gemv_glu_eligible(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dim() == 2 and a.shape[0] <= GEMV_GLU_MAX_M and w.dtype == torch.bfloat16 and a.dtype in SEQ_DTYPE and a.shape[1] % 32 == 0
            and a.stride(1) == 1 and (a.stride(0) * a.element_size()) % 16 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def dense_gemv_glu(a: torch.Tensor, w_pairs: torch.Tensor, limit: float | None, slope: float, up_shift: float, out_dtype=torch.float32) -> torch.Tensor:
    """Decode-sized GLU front half in one launch (ktx_dense_gemv_glu): a [M <= 16, K] x w_pairs [2F, K] (bf16, rows alternating gate_f,
    up_f) -> g sigmoid(slope g) (u + up_shift) with the bounded g, u; [M, F] of out_dtype."""
    if not dense_gemv_glu_eligible(a, w_pairs) or not w_pairs.is_contiguous() or w_pairs.shape[1] != a.shape[1] or w_pairs.shape[0] % 2:
        raise KtxError(f"dense_gemv_glu: {a.dtype} {tuple(a.shape)} x {w_pairs.dtype} {tuple(w_pairs.shape)}^T does not fit")
    M, K = a.shape
    Fh = w_pairs.shape[0] // 2
    out = torch.empty((M, Fh), dtype=out_dtype, device=a.device)
    check(lib.ktx_dense_gemv_glu(M, Fh, K, a.data_ptr(), SEQ_DTYPE[a.dtype], a.stride(0), w_pairs.data_ptr(), out.data_ptr(), SEQ_DTYPE[out_dtype],
                                 out.stride(0), float("inf") if limit is None else float(limit), float(slope), float(up_shift),
                                 _stream_ptr(a.device)))
    return out


def dense_gemm_skinny(a: torch.Tensor, w: torch.Tensor, act: str | None = None) -> torch.Tensor:
    """dense_gemm with an fp32 result for products with FEW output columns (a router, a low-rank projection): on prompt-sized steps their
    64 x 64 tiles are too few to fill the chip, so K is split over workgroups that add into a zeroed result (fp32 atomics: the order of
    the partial sums, and with it the last bit, is not fixed); the activation then has its own launch."""
    M, K = a.shape
    N = w.shape[0]
    tiles = ((M + 63) // 64) * ((N + 63) // 64)
    ks = 1
    if M >= SKINNY_MIN_M and tiles < 256:
        while ks < 8 and tiles * ks * 2 <= 512 and K // (ks * 2) >= 256:
            ks *= 2
    if ks == 1:
        return dense_gemm(a, w, act=act)
    y = dense_gemm(a, w, ksplit=ks)
    if ACT[act]:
        check(lib.ktx_gelu_tanh(y.numel(), y.data_ptr(), SEQ_DTYPE[y.dtype], _stream_ptr(y.device)))
    return y


LIBRARY_GEMM_MIN_M = 64
SKINNY_MIN_M = 256
_LIBRARY_GEMM: list = []


def _library_gemm():
    """ktransformers_amd._native.gemm_bf16_nt when the whole library is built, else None (libktx_seq.so alone: ktx_dense_gemm serves)."""
    if not _LIBRARY_GEMM:
        fn = None
        if os.path.exists(LIB_PATHS[0]) and not os.environ.get("KTX_SEQ_OWN_GEMM"):
            try:
                from ktransformers_amd._native import gemm_bf16_nt as fn
            except Exception:
                fn = None
        _LIBRARY_GEMM.append(fn)
    return _LIBRARY_GEMM[0]


def sigattn_config(heads: int, kv_heads: int, dim: int, scale: float, temp_coef: float, temp_every: int, slope_span: float,
                   page_size: int, cache_dtype) -> _SigAttnConfig:
    return _SigAttnConfig(heads, kv_heads, dim, float(scale), float(temp_coef), int(temp_every), float(slope_span), int(page_size),
                          SEQ_DTYPE[cache_dtype])


def sigattn_prep(cfg: _SigAttnConfig, proj: torch.Tensor, q_off: int, k_off: int, wq: torch.Tensor, wk: torch.Tensor, eps: float,
                 positions: torch.Tensor, cache_loc: torch.Tensor, kcache: torch.Tensor, kinv: torch.Tensor) -> torch.Tensor:
    """proj fp32 [T, *]; returns the folded queries fp32 [T, heads, dim]; appends key rows + 1/rms to the cache (ktx_sigattn_prep)."""
    T = proj.shape[0]
    _seq_dev(positions, torch.int32, "sigattn_prep positions"), _seq_dev(cache_loc, torch.int32, "sigattn_prep cache_loc")
    if proj.dtype != torch.float32 or proj.stride(1) != 1 or positions.numel() != T or cache_loc.numel() != T:
        raise KtxError("sigattn_prep: proj must be fp32 rows with one position and cache row per token")
    q = torch.empty((T, cfg.heads, cfg.dim), dtype=torch.float32, device=proj.device)
    check(lib.ktx_sigattn_prep(C.byref(cfg), T, proj.data_ptr(), proj.stride(0), q_off, k_off, wq.data_ptr(), wk.data_ptr(), float(eps),
                               positions.data_ptr(), cache_loc.data_ptr(), kcache.data_ptr(), kinv.data_ptr(), q.data_ptr(),
                               _stream_ptr(proj.device)))
    return q


def sigattn_forward(cfg: _SigAttnConfig, q: torch.Tensor, kcache: torch.Tensor, kinv: torch.Tensor, tok_req: torch.Tensor,
                    positions: torch.Tensor, page_indptr: torch.Tensor, page_indices: torch.Tensor, pb: torch.Tensor,
                    talk: torch.Tensor, nsplit: int = 1, out_dtype=torch.float32) -> torch.Tensor:
    """-> [T, heads * dim] of out_dtype (ktx_sigattn_forward)."""
    T = q.shape[0]
    for t, what in ((tok_req, "tok_req"), (positions, "positions"), (page_indptr, "page_indptr"), (page_indices, "page_indices")):
        _seq_dev(t, torch.int32, "sigattn_forward " + what)
    _seq_dev(q, torch.float32, "sigattn_forward q")
    HD = cfg.heads * cfg.dim
    out = torch.empty((T, HD), dtype=out_dtype, device=q.device)
    partial = torch.empty((nsplit, T, HD), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_sigattn_forward(C.byref(cfg), T, q.data_ptr(), kcache.data_ptr(), kinv.data_ptr(), tok_req.data_ptr(), positions.data_ptr(),
                                  page_indptr.data_ptr(), page_indices.data_ptr(), pb.data_ptr(), talk.data_ptr(), int(nsplit),
                                  partial.data_ptr() if partial is not None else None, out.data_ptr(), SEQ_DTYPE[out_dtype],
                                  _stream_ptr(q.device)))
    return out


def sigattn_prefill_eligible(cfg: _SigAttnConfig) -> bool:
    return bool(lib.ktx_sigattn_prefill_eligible(C.byref(cfg)))


def sigattn_prefill(cfg: _SigAttnConfig, q: torch.Tensor, kcache: torch.Tensor, kinv: torch.Tensor, q_indptr: torch.Tensor,
                    pos0: torch.Tensor, page_indptr: torch.Tensor, page_indices: torch.Tensor, pb: torch.Tensor, talk: torch.Tensor,
                    max_q_len: int, nsplit: int = 1) -> torch.Tensor:
    """The matrix-core kernel, prompts and decode steps (ktx_sigattn_prefill) -> bf16 [T, heads * dim]."""
    for t, what in ((q_indptr, "q_indptr"), (pos0, "pos0"), (page_indptr, "page_indptr"), (page_indices, "page_indices")):
        _seq_dev(t, torch.int32, "sigattn_prefill " + what)
    _seq_dev(q, torch.float32, "sigattn_prefill q")
    T, HD = q.shape[0], cfg.heads * cfg.dim
    out = torch.empty((T, HD), dtype=torch.bfloat16, device=q.device)
    partial = torch.empty((nsplit, T, HD), dtype=torch.float32, device=q.device) if nsplit > 1 else None
    check(lib.ktx_sigattn_prefill(C.byref(cfg), pos0.numel(), T, int(max_q_len), q.data_ptr(), kcache.data_ptr(), kinv.data_ptr(),
                                  q_indptr.data_ptr(), pos0.data_ptr(), page_indptr.data_ptr(), page_indices.data_ptr(), pb.data_ptr(),
                                  talk.data_ptr(), int(nsplit), partial.data_ptr() if partial is not None else None, out.data_ptr(),
                                  _stream_ptr(q.device)))
    return out


def mlstm_config(heads: int, dim: int, vdim: int, gate_cap: float, eps: float, denom_eps: float = 1e-6) -> _MlstmConfig:
    return _MlstmConfig(heads, dim, vdim, float(gate_cap), float(eps), float(denom_eps))


def mlstm_forward(cfg: _MlstmConfig, proj: torch.Tensor, offs: dict, ib: torch.Tensor, fb: torch.Tensor, q_indptr: torch.Tensor,
                  pos0: torch.Tensor, slot: torch.Tensor, S: torch.Tensor, n: torch.Tensor, m: torch.Tensor,
                  max_q_len: int | None = None) -> torch.Tensor:
    """The recurrence over the flattened batch (ktx_mlstm_forward); offs = column offsets of q, k, v, i, f in proj's rows.
    Returns the un-normed outputs fp32 [T, heads * vdim]; the state tensors are updated in place."""
    for t, what in ((q_indptr, "q_indptr"), (pos0, "pos0"), (slot, "slot")):
        _seq_dev(t, torch.int32, "mlstm_forward " + what)
    for t, what in ((S, "S"), (n, "n"), (m, "m"), (ib, "ib"), (fb, "fb")):
        _seq_dev(t, torch.float32, "mlstm_forward " + what)
    if proj.dtype != torch.float32 or proj.stride(1) != 1:
        raise KtxError("mlstm_forward: proj must be fp32 rows")
    B, T = slot.numel(), proj.shape[0]
    o = torch.empty((T, cfg.heads * cfg.vdim), dtype=torch.float32, device=proj.device)
    gates = torch.empty(((B + 8 * T) * cfg.heads,), dtype=torch.float32, device=proj.device)
    check(lib.ktx_mlstm_forward(C.byref(cfg), B, q_indptr.data_ptr(), pos0.data_ptr(), slot.data_ptr(), proj.data_ptr(), proj.stride(0),
                                offs["q"], offs["k"], offs["v"], offs["i"], offs["f"], ib.data_ptr(), fb.data_ptr(), S.data_ptr(),
                                n.data_ptr(), m.data_ptr(), gates.data_ptr(), o.data_ptr(), int(T if max_q_len is None else max_q_len),
                                _stream_ptr(proj.device)))
    return o


def mlstm_gate_norm(cfg: _MlstmConfig, o_raw: torch.Tensor, proj: torch.Tensor, g_off: int, w: torch.Tensor, out_dtype) -> torch.Tensor:
    T = o_raw.shape[0]
    out = torch.empty((T, cfg.heads * cfg.vdim), dtype=out_dtype, device=o_raw.device)
    check(lib.ktx_mlstm_gate_norm(C.byref(cfg), T, o_raw.data_ptr(), proj.data_ptr(), proj.stride(0), g_off, w.data_ptr(), out.data_ptr(),
                                  SEQ_DTYPE[out_dtype], _stream_ptr(o_raw.device)))
    return out


def rms_combine(y1: torch.Tensor, wn: torch.Tensor | None, eps: float, one_plus: bool = False, residual: torch.Tensor | None = None,
                y2: torch.Tensor | None = None, w1: torch.Tensor | None = None, w2: torch.Tensor | None = None,
                rows: torch.Tensor | None = None, out_dtype=torch.float32) -> torch.Tensor:
    """ktx_rms_combine: z = y2 is None ? y1 : half the sum of the unit-RMS inputs times their weights; r = unit-RMS(z) * wn (or 1 + wn);
    `residual += r` in place (returned) or a new [T, W] tensor of out_dtype.  rows: int32 gather of y1's rows."""
    _seq_dev(y1, torch.float32, "rms_combine y1")
    W = y1.shape[-1]
    T = rows.numel() if rows is not None else y1.numel() // W
    for t in (y2, w1, w2, wn, residual):
        if t is not None:
            _seq_dev(t, torch.float32, "rms_combine")
    out = None if residual is not None else torch.empty((T, W), dtype=out_dtype, device=y1.device)
    check(lib.ktx_rms_combine(T, W, y1.data_ptr(), w1.data_ptr() if w1 is not None else None, y2.data_ptr() if y2 is not None else None,
                              w2.data_ptr() if w2 is not None else None, wn.data_ptr() if wn is not None else None, 1 if one_plus else 0,
                              float(eps), residual.data_ptr() if residual is not None else None,
                              rows.data_ptr() if rows is not None else None, out.data_ptr() if out is not None else None,
                              SEQ_DTYPE[out_dtype], _stream_ptr(y1.device)))
    return residual if residual is not None else out
