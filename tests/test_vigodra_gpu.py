"""Vigodra on the GPU against the plain CPU statement of the design (oracle/vigodra_ref.py, fp64): every mechanism alone through its
kernels and operator, then the model through the framework's registry, cache manager, step function and generation loops — whole
prompts, token-by-token decoding, portions, unequal batches, reused pages and slots, keys at the window's edge, among the kept first
tokens and at page borders, odd sizes.  Small random configurations; fp32 runs are held to rounding, bf16 runs to bf16 rounding."""
import math

import pytest
import torch

from oracle import vigodra_ref as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 3e-4, BF16: 6e-2}


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def rows_rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float(((got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)).max())


def build(cfg, seed, dtype, max_tokens=2048, max_requests=8, page_size=16, P=None):
    from ktransformers_amd.models import load_model
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_vigodra import vigodra_layer_specs
    from ktransformers_amd.util.loader import DictLoader
    P = R.random_checkpoint(cfg, seed) if P is None else P
    model, config, _ = load_model(cfg, dtype=dtype, device=DEV, loader=DictLoader(P))
    cache = KHybridCache(vigodra_layer_specs(config), max_tokens, max_requests=max_requests, page_size=page_size, dtype=dtype, device=DEV)
    return model, cache, R.as_double(P)


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def engine_of(model, cache, **kw):
    from ktransformers_amd.util.batch_engine import BatchEngine
    return BatchEngine(model, cache, **kw)


def steps(eng, rid, toks, sizes, end=True):
    """Feed toks in portions of the given sizes; logits of every position."""
    got, at = [], 0
    for n in sizes:
        last = at + n == len(toks)
        got.append(eng.step([{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}], [rid] if last and end else []))
        at += n
    assert at == len(toks)
    return torch.cat(got)


def batch_of(cache, entries):
    for rid, _ in entries:
        if rid not in cache.requests:
            cache.admit(rid)
    return cache.plan(entries)


# ---- the element-wise kernels and the norm ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("W,levels,lp", [(32, 0, None), (48, 1, BF16), (260, 4, BF16), (1024, 11, F32), (7, 3, None), (1500, 2, BF16),
                                         (4096, 3, None), (4100, 2, BF16)])
def test_post_norm_with_scaled_residual_and_depth_average(W, levels, lp):
    """ktx_postnorm_mix against the plain layer norm and weighted sum: with and without the sublayer's output, its bias, the stack and the
    average; in place and out of place; a low-precision copy; rows held in registers (up to 4096 entries) and in LDS (beyond)."""
    from ktransformers_amd._native_hyb import postnorm_mix
    g = torch.Generator().manual_seed(W + levels)
    T, alpha, eps = 5, 2.25, 1e-5
    x, y = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g)
    w, b, yb = 1 + 0.3 * torch.randn(W, generator=g), torch.randn(W, generator=g), torch.randn(W, generator=g)
    stack = torch.randn(levels + 1, T, W, generator=g) if levels else None
    dwa = torch.randn(levels + 1, generator=g) if levels else None
    for use_y, use_b, use_dwa, inplace in ((True, True, True, True), (True, False, True, False), (False, True, False, True), (False, False, True, False)):
        v = R.layer_norm(alpha * x.double() + (y.double() if use_y else 0) + (yb.double() if use_b else 0), w.double(), b.double(), eps)
        want = v
        if stack is not None and use_dwa:
            want = sum(dwa[j].double() * stack[j].double() for j in range(levels)) + dwa[levels].double() * v
        xin = x.clone().to(DEV)
        xout = xin if inplace else torch.full((T, W), float("nan"), device=DEV)
        st = stack.clone().to(DEV) if stack is not None else None
        got = postnorm_mix(xin, xout, w.to(DEV), b.to(DEV), eps, alpha=alpha, y=y.to(DEV) if use_y else None, ybias=yb.to(DEV) if use_b else None,
                           stack=st, level=levels, dwa=dwa.to(DEV) if stack is not None and use_dwa else None, lp_dtype=lp)
        assert rel(xout, want) < 2e-6
        assert rel(got, want) < (2e-6 if lp in (None, F32) else 4e-3) and got.dtype == (lp or F32)
        if st is not None:
            assert rel(st[levels], v) < 2e-6 and torch.equal(st[:levels].cpu(), stack[:levels])
        if not inplace:
            assert torch.equal(xin.cpu(), x)


def test_post_norm_may_read_a_level_of_the_stack_it_writes_to():
    from ktransformers_amd._native_hyb import postnorm_mix
    g = torch.Generator().manual_seed(3)
    T, W = 4, 40
    stack = torch.randn(3, T, W, generator=g).to(DEV)
    keep = stack.clone()
    w, b, dwa = torch.ones(W, device=DEV), torch.zeros(W, device=DEV), torch.tensor([0.5, -1.0], device=DEV)
    x = torch.empty(T, W, device=DEV)
    postnorm_mix(stack[0], x, w, b, 1e-6, alpha=1.0, stack=stack, level=1, dwa=dwa)
    v = R.layer_norm(keep[0].double().cpu(), 1.0, 0.0, 1e-6)
    assert rel(x, 0.5 * keep[0].double().cpu() - v) < 2e-6 and torch.equal(stack[0], keep[0]) and torch.equal(stack[2], keep[2])


@pytest.mark.parametrize("limit", [0.75, 2.0, None])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_bounded_glu_activation_and_sigmoid_gate(limit, dtype):
    from ktransformers_amd._native_hyb import glu_clamp_rows, sigmoid_gate_rows
    g = torch.Generator().manual_seed(5)
    gu = torch.randn(9, 2 * 37, generator=g) * 2
    gate, up = gu[:, :37].double(), gu[:, 37:].double()
    if limit is not None:
        gate, up = gate.clamp(max=limit), up.clamp(-limit, limit)
    want = gate * torch.sigmoid(1.702 * gate) * (up + 1.0)
    got = glu_clamp_rows(gu.to(DEV), limit, 1.702, 1.0, out_dtype=dtype)
    assert rel(got, want) < (1e-6 if dtype == F32 else 4e-3)
    pairs = torch.stack([gu[:, :37], gu[:, 37:]], dim=2).reshape(9, 74)          # gate_0, up_0, gate_1, up_1, ...
    got = glu_clamp_rows(pairs.to(DEV), limit, 1.702, 1.0, out_dtype=dtype, paired=True)
    assert rel(got, want) < (1e-6 if dtype == F32 else 4e-3)
    wide = torch.randn(9, 100, generator=g)
    o = torch.randn(9, 37, generator=g).to(dtype)
    got = sigmoid_gate_rows(o.to(DEV), wide.to(DEV)[:, 11:48], out_dtype=dtype)
    assert rel(got, o.double() * torch.sigmoid(wide[:, 11:48].double())) < (1e-6 if dtype == F32 else 4e-3)


@pytest.mark.parametrize("M,F,K,limit", [(1, 40, 64, 1.5), (8, 37, 96, None), (16, 16, 32, 0.5), (3, 300, 2048, 7.0)])
@pytest.mark.parametrize("a_dtype,out_dtype", [(F32, F32), (BF16, BF16), (F32, BF16)])
def test_decode_sized_glu_product_with_the_activation_in_its_launch(M, F, K, limit, a_dtype, out_dtype):
    from ktransformers_amd._native_seq import dense_gemv_glu, dense_gemv_glu_eligible
    g = torch.Generator().manual_seed(M + F)
    a = torch.randn(M, K, generator=g).to(BF16)
    gate, up = (torch.randn(F, K, generator=g) * 2 / math.sqrt(K)).to(BF16), (torch.randn(F, K, generator=g) * 2 / math.sqrt(K)).to(BF16)
    gv, uv = a.double() @ gate.double().T, a.double() @ up.double().T
    if limit is not None:
        gv, uv = gv.clamp(max=limit), uv.clamp(-limit, limit)
    want = gv * torch.sigmoid(1.702 * gv) * (uv + 1.0)
    w = torch.stack([gate, up], dim=1).reshape(2 * F, K).contiguous().to(DEV)
    ad = a.to(a_dtype).to(DEV)
    assert dense_gemv_glu_eligible(ad, w) and not dense_gemv_glu_eligible(torch.zeros(17, K, dtype=a_dtype, device=DEV), w)
    got = dense_gemv_glu(ad, w, limit, 1.702, 1.0, out_dtype=out_dtype)
    assert rel(got, want) < (2e-5 if out_dtype == F32 else 4e-3)


def test_distance_rows_follow_the_plain_bucket_rule():
    from ktransformers_amd.operators.window_attention import KWindowGQAttention
    for rows, far in ((16, 100), (8, 20), (32, 256), (4, 3.5), (2, 2), (12, 1000), (6, 81)):
        got = KWindowGQAttention.distance_rows(rows, far)
        assert got == [R.distance_bucket(n, rows, far) for n in range(len(got))] and got[-1] == rows - 1 and len(got) >= far
        assert R.distance_bucket(10 ** 6, rows, far) == rows - 1


# ---- attention kernels with hand-made queries, keys and values: one key made to stand out -----------------------------------------
def run_swa(H, G, D, V, T, window, keep, rel_t, far, sink, q, k, v, dtype, kernel, nsplit=1, page_size=8, t_new=None):
    """The attention kernels on keys and values written straight into paged caches; the last t_new positions are the queries."""
    from ktransformers_amd._native_swa import swa_config, swa_forward, swa_mfma, swa_mfma_eligible
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.operators.window_attention import KWindowGQAttention
    cache = KHybridCache([{"kv": (G, D, V)}], 4 * T + 64, max_requests=4, page_size=page_size, dtype=dtype, device=DEV)
    cache.admit("pad"), cache.plan([("pad", page_size + 3)])          # the request's pages do not start at row 0
    t_new = T if t_new is None else t_new
    cache.admit("r")
    if T > t_new:
        cache.plan([("r", T - t_new)])
    b = cache.plan([("r", t_new)])
    pages = cache.requests["r"]["pages"]
    loc = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in range(T)], device=DEV)
    cache.k_caches[0][loc] = k.to(DEV).to(dtype)
    cache.v_caches[0][loc] = v.to(DEV).to(dtype)
    dist = None
    if rel_t is not None:
        dist = rel_t.float().to(DEV)[torch.tensor(KWindowGQAttention.distance_rows(rel_t.shape[0], far), device=DEV)].contiguous()
    cfg = swa_config(H, G, D, V, 0, False, False, 1e-6, 1.0, window or 0, page_size, dtype, keep_first=keep,
                     bias_span=0 if dist is None else dist.shape[0] - 1)
    qn = q[T - t_new:].reshape(t_new, H * D).float().contiguous().to(DEV)
    sk = None if sink is None else sink.float().to(DEV)
    if kernel == "mfma":
        assert swa_mfma_eligible(cfg)
        return swa_mfma(cfg, qn, cache.k_caches[0], cache.v_caches[0], b, sk, None, nsplit=nsplit, out_dtype=F32, dist_bias=dist)
    return swa_forward(cfg, qn, cache.k_caches[0], cache.v_caches[0], b, sk, None, nsplit=nsplit, out_dtype=F32, dist_bias=dist)


SWA_CASES = [
    # H, G, D, V, T, window, keep, table rows, far, sink
    (4, 2, 32, 16, 70, 12, 3, 8, 20, True),
    (3, 1, 10, 6, 45, 7, 0, 6, 30, True),          # odd sizes: the vector-ALU form only
    (6, 2, 64, 80, 150, 40, 5, 12, 60, True),
    (2, 2, 32, 48, 90, None, 0, 4, 9, False),      # no window, no sink
    (4, 4, 64, 128, 130, 33, 40, None, None, True),  # more kept tokens than the window is wide, no distance table
    (6, 2, 32, 112, 64, 1, 1, 2, 2, False),        # a window of one token plus one kept token
]


@pytest.mark.parametrize("case", SWA_CASES)
@pytest.mark.parametrize("kernel,dtype", [("valu", F32), ("valu", BF16), ("mfma", BF16)])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_biased_window_attention_kernels(case, kernel, dtype, nsplit):
    H, G, D, V, T, window, keep, rows, far, use_sink = case
    if kernel == "mfma" and (D % 32 or V % 16):
        pytest.skip("sizes the matrix-core form does not take")
    g = torch.Generator().manual_seed(T)
    q, k, v = (torch.randn(T, n, d, generator=g).to(dtype).double() for n, d in ((H, D), (G, D), (G, V)))
    q = q * D ** -0.5
    rel_t = (torch.randn(rows, H, generator=g) * 2).to(BF16).double() if rows else None
    sink = torch.randn(H, generator=g).double() if use_sink else None
    want = R.attention_core(q, k, v, 1.0, window, keep, rel_t, far, sink)
    for t_new in (T, 1, 5):
        got = run_swa(H, G, D, V, T, window, keep, rel_t, far, sink, q, k, v, dtype, kernel, nsplit=nsplit, t_new=t_new)
        assert rel(got.view(t_new, H, V), want[T - t_new:]) < (2e-5 if kernel == "valu" else 1.5e-2), t_new


@pytest.mark.parametrize("kernel,dtype", [("valu", F32), ("mfma", BF16)])
@pytest.mark.parametrize("t_new", [None, 1, 2])
def test_one_boosted_key_at_the_edges_of_window_and_kept_tokens(kernel, dtype, t_new):
    """ONE key with a score far above the rest: just inside the window it takes all the weight, just outside none; the last kept token
    stays visible however far back, the first token behind the kept ones does not; also with the key on either side of a page border."""
    H, G, D, V, T, window, keep, ps = 2, 1, 32, 16, 83, 24, 5, 8
    g = torch.Generator().manual_seed(11)
    base_q, base_k = torch.randn(T, H, D, generator=g) * 0.05, torch.randn(T, G, D, generator=g) * 0.05
    v = torch.randn(T, G, V, generator=g).to(BF16).double()
    i = T - 1
    for j, seen in ((i - window + 1, True), (i - window, False), (keep - 1, True), (keep, False), (0, True), (i, True),
                    (i - window + 1 + (ps - (i - window + 1) % ps) % ps, True), (i - 16, True), (i - 17, True)):
        q, k = base_q.clone(), base_k.clone()
        u = torch.zeros(D)
        u[3] = 1.0
        q[i, :, :] = 6.0 * u
        k[j, 0, :] = 6.0 * u                                   # score 36 against ~0 elsewhere
        q, k = q.to(BF16).double(), k.to(BF16).double()
        want = R.attention_core(q, k, v, 1.0, window, keep, None, None, torch.zeros(H, dtype=torch.float64))
        hit = float((want[i, 0] - v[j, 0]).abs().max()) < 1e-6
        assert hit == seen, (j, seen)                           # the plain statement itself tells the cases apart
        n = T if t_new is None else t_new
        got = run_swa(H, G, D, V, T, window, keep, None, None, torch.zeros(H), q, k, v, dtype, kernel, page_size=ps, t_new=n)
        assert rel(got.view(n, H, V), want[T - n:]) < (2e-5 if kernel == "valu" else 1.5e-2), (j, seen)
        assert (float((got.view(n, H, V)[-1, 0].double().cpu() - v[j, 0]).abs().max()) < 2e-2) == seen


@pytest.mark.parametrize("kernel,dtype", [("valu", F32), ("mfma", BF16)])
def test_distance_bias_decides_between_equal_keys(kernel, dtype):
    """All keys equal, so only the learned bias by distance tells them apart: a large entry in ONE row of the table moves the weight to
    exactly the distances of that row — the rows' edges, the far end and the last row beyond it."""
    H, G, D, V, T, rows, far = 2, 1, 32, 16, 140, 8, 50
    k = torch.ones(T, G, D, dtype=torch.float64) * 0.1
    q = torch.ones(T, H, D, dtype=torch.float64) * 0.1
    v = torch.eye(T, dtype=torch.float64)[:, :V].clone().view(T, G, V)
    v[:, 0, :] = torch.randn(T, V, generator=torch.Generator().manual_seed(2)).to(BF16).double()
    for row in range(rows):
        rel_t = torch.zeros(rows, H, dtype=torch.float64)
        rel_t[row, 0] = 30.0
        want = R.attention_core(q, k, v, 1.0, None, 0, rel_t, far, None)
        dists = [n for n in range(T) if R.distance_bucket(n, rows, far) == row]
        i = T - 1
        assert rel(want[i, 0], torch.stack([v[i - n, 0] for n in dists]).mean(0)) < 1e-9
        for t_new in (T, 1):
            got = run_swa(H, G, D, V, T, None, 0, rel_t, far, None, q, k, v, dtype, kernel, t_new=t_new)
            assert rel(got.view(t_new, H, V), want[T - t_new:]) < (2e-5 if kernel == "valu" else 1.5e-2), row


def run_latent(H, L, R, T, window, scale, q, rows, dtype, kernel, nsplit=1, page_size=8, t_new=None):
    """The latent-attention kernels (no sink) on rows written straight into a paged cache; the last t_new positions are the queries."""
    from ktransformers_amd._native_hyb import latattn_config, latattn_forward, latattn_mfma, latattn_mfma_eligible
    from ktransformers_amd.models.custom_cache import KHybridCache
    cache = KHybridCache([{"latent": L + R}], 4 * T + 64, max_requests=4, page_size=page_size, dtype=dtype, device=DEV)
    cache.admit("pad"), cache.plan([("pad", page_size + 3)])
    t_new = T if t_new is None else t_new
    cache.admit("r")
    if T > t_new:
        cache.plan([("r", T - t_new)])
    b = cache.plan([("r", t_new)])
    pages = cache.requests["r"]["pages"]
    loc = torch.tensor([pages[p // page_size] * page_size + p % page_size for p in range(T)], device=DEV)
    cache.lat_caches[0][loc] = rows.to(DEV).to(dtype)
    cfg = latattn_config(H, 8, R, 8, L, 0, scale, window or 0, 1e-6, page_size, dtype)
    qn = q[T - t_new:].reshape(t_new, H * (L + R)).float().contiguous().to(DEV)
    if kernel == "mfma":
        assert latattn_mfma_eligible(cfg)
        return latattn_mfma(cfg, qn, cache.lat_caches[0], b, None, nsplit=nsplit, out_dtype=F32)
    return latattn_forward(cfg, qn, cache.lat_caches[0], b, None, nsplit=nsplit, out_dtype=F32)


@pytest.mark.parametrize("kernel,dtype,L,Rd", [("valu", F32, 24, 6), ("valu", BF16, 9, 4), ("mfma", BF16, 64, 16)])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_latent_attention_without_a_sink_and_its_window_edge(kernel, dtype, L, Rd, nsplit):
    """An ordinary softmax over the window (no extra term in the denominator): random rows, then ONE boosted row just inside and just
    outside the window, at position 0 and on either side of a page border — as prompts, single decode tokens and portions of two."""
    H, T, window, ps = 3, 77, 20, 8
    g = torch.Generator().manual_seed(L)
    q = (torch.randn(T, H, L + Rd, generator=g) * (L + Rd) ** -0.5).to(dtype).double()
    rows = torch.randn(T, L + Rd, generator=g).to(dtype).double()
    tol = 2e-5 if kernel == "valu" else 1.5e-2
    want = R.latent_core(q, rows, L, 1.0, window)
    for t_new in (T, 1, 2):
        got = run_latent(H, L, Rd, T, window, 1.0, q, rows, dtype, kernel, nsplit=nsplit, page_size=ps, t_new=t_new)
        assert rel(got.view(t_new, H, L), want[T - t_new:]) < tol, t_new
    i = T - 1
    for j, seen in ((i - window + 1, True), (i - window, False), (0, False), (i, True), (i - 13, True), (i - 12, True)):
        qb, rb = q.clone() * 0.05, rows.clone()
        rb[:, 2] *= 0.05
        qb[i, :, :] = 0.0
        qb[i, :, 2] = 6.0
        rb[j, 2] = 6.0                                          # score 36 against ~0 elsewhere
        qb, rb = qb.to(dtype).double(), rb.to(dtype).double()
        want = R.latent_core(qb, rb, L, 1.0, window)
        assert (float((want[i, 0] - rb[j, :L]).abs().max()) < 1e-6) == seen, j
        for t_new in (T, 1, 2):
            got = run_latent(H, L, Rd, T, window, 1.0, qb, rb, dtype, kernel, nsplit=nsplit, page_size=ps, t_new=t_new)
            assert rel(got.view(t_new, H, L), want[T - t_new:]) < tol, (j, t_new)
            assert (float((got.view(t_new, H, L)[-1, 0].double().cpu() - rb[j, :L]).abs().max()) < 3e-2) == seen, (j, t_new)


# ---- the attention operators alone (a one-layer model without feed-forward reads its mixer's input from the embedding) -------------
def mixer_alone(layer, dtype, seed, T=40, width=32, **kw):
    """The layer's mixer through the model: logits of a one-layer model whole, token by token and in portions, against the statement."""
    layer = dict(layer, mlp=None)
    cfg = R.make_config([layer], width=width)
    model, cache, P = build(cfg, seed, dtype, page_size=8, **kw)
    toks = tokens_of(cfg, T, seed)
    want = R.forward(P, cfg, toks)
    eng = engine_of(model, cache)
    tol = 3e-4 if dtype == F32 else 5e-2
    for sizes in ([T], [1] * T, [T - 9, 2, 2, 5], [3, T - 3], [2] * (T // 2) + [1] * (T % 2)):
        assert rows_rel(steps(eng, "a", toks, sizes), want) < tol, sizes
    return model


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("layer", [
    R.attention_layer(),
    R.attention_layer(heads=3, kv_heads=1, dim=10, vdim=6, window=5, keep_first=0, conv=2, bias_max=7, scale=0.4),
    R.attention_layer(heads=4, kv_heads=1, dim=32, vdim=80, window=9, keep_first=4, conv=4, bias_max=33),
    R.attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, window=None, conv=0, bias_max=None),
    R.attention_layer(heads=2, kv_heads=1, dim=64, vdim=16, window=3, keep_first=1, conv=1, bias_max=5),
    R.attention_layer(heads=1, kv_heads=1, dim=1, vdim=1, window=1, keep_first=1, conv=9, bias_max=4),
], ids=["plain", "odd", "mfma-80", "bare", "one-tap", "ones"])
def test_biased_window_attention_layer(layer, dtype):
    model = mixer_alone(layer, dtype, 3)
    assert type(model.l0.mix).__name__ == "KWindowGQAttention" and model.l0.mix.conv_form


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("layer", [
    R.latent_layer(),
    R.latent_layer(heads=3, dim=5, rot_dim=6, vdim=7, kv_rank=9, window=4, rot_dims=4, base=77.0),
    R.latent_layer(heads=4, dim=16, rot_dim=16, vdim=24, kv_rank=64, window=11),            # sizes the matrix-core form takes
    R.latent_layer(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=128, window=None),
    R.latent_layer(heads=1, dim=1, rot_dim=2, vdim=1, kv_rank=1, window=1),
], ids=["plain", "odd", "mfma-64", "mfma-128-full", "ones"])
def test_gated_latent_attention_layer(layer, dtype):
    model = mixer_alone(layer, dtype, 4)
    assert model.l0.mix.rot_half and not model.l0.mix.has_sink and model.l0.mix.gated


def test_rotate_half_differs_from_neighbour_pairs():
    """The statement's rotation pairs entry i with i + dims / 2: a model loaded with the neighbour-pair layout must NOT agree."""
    cfg = R.make_config([R.latent_layer(mlp=None)])
    model, cache, P = build(cfg, 5, F32, page_size=8)
    toks = tokens_of(cfg, 20, 1)
    want = R.forward(P, cfg, toks)
    assert rows_rel(steps(engine_of(model, cache), "a", toks, [20]), want) < 3e-4
    object.__setattr__(model.l0.mix, "rot_half", False)
    model.l0.mix._cfg.clear()
    assert rows_rel(steps(engine_of(model, cache), "b", toks, [20]), want) > 1e-2


# ---- the model ------------------------------------------------------------------------------------------------------------------
CONFIGS = {
    # both mixers, a shared latent cache, a layer without feed-forward
    "mixed": lambda: R.make_config([R.latent_layer(), R.attention_layer(), R.attention_layer(heads=2, kv_heads=2, window=7, keep_first=3, mlp=None),
                                    R.latent_layer(kv_from=0, window=6)]),
    # attention first, two latent groups, the sharing layers not directly behind their sources, odd sizes everywhere
    "odd": lambda: R.make_config([R.attention_layer(heads=3, kv_heads=1, dim=10, vdim=6, window=5, keep_first=1, conv=2, bias_max=9, scale=0.7,
                                                    mlp=R.dense_mlp(ff=7, limit=0.6)),
                                  R.latent_layer(heads=3, dim=5, rot_dim=6, vdim=7, kv_rank=9, window=4, rot_dims=4, base=77.0),
                                  R.latent_layer(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5, window=20, mlp=None),
                                  R.latent_layer(heads=2, dim=3, rot_dim=6, vdim=5, kv_rank=9, window=9, rot_dims=4, base=77.0, kv_from=1),
                                  R.latent_layer(heads=5, dim=2, rot_dim=2, vdim=2, kv_rank=5, window=3, kv_from=2, mlp=R.dense_mlp(ff=3, limit=5.0))],
                                 width=29, vocab=53, eps=1e-3, alpha=0.8, scale=1.3),
    # sizes the matrix-core kernels take
    "wide": lambda: R.make_config([R.latent_layer(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, window=40),
                                   R.attention_layer(heads=8, kv_heads=2, dim=32, vdim=48, window=24, keep_first=5, conv=4, bias_max=50),
                                   R.latent_layer(heads=2, dim=16, rot_dim=16, vdim=64, kv_rank=64, window=17, kv_from=0),
                                   R.attention_layer(heads=4, kv_heads=4, dim=64, vdim=16, window=100, keep_first=0, conv=3, bias_max=30)],
                                  width=128, vocab=97),
    # everything optional left out: no window, no convolution, no distance table, no limit, no feed-forward
    "bare": lambda: R.make_config([R.attention_layer(window=None, conv=0, bias_max=None, mlp=None), R.latent_layer(window=None, mlp=R.dense_mlp(limit=None))],
                                  alpha=1.0, scale=1.0),
    # sizes that are 1
    "ones": lambda: R.make_config([R.attention_layer(heads=1, kv_heads=1, dim=1, vdim=1, window=1, keep_first=1, conv=1, bias_max=2, mlp=R.dense_mlp(ff=1)),
                                   R.latent_layer(heads=1, dim=1, rot_dim=2, vdim=1, kv_rank=1, window=1)], width=3, vocab=5),
}


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_model_whole_decoded_and_in_portions(name, dtype):
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 7, dtype, page_size=16)
    T = 61
    toks = tokens_of(cfg, T, 9)
    want, layers = R.forward(P, cfg, toks, return_layers=True)
    b = batch_of(cache, [("L", T)])
    lg, trail = model(torch.tensor(toks, dtype=torch.int32, device=DEV), None, cache, batch=b, return_layers=True)
    cache.release("L")
    tol = TOL[dtype]
    for i in range(len(cfg["layers"])):
        assert rel(trail[i], layers[i]) < (tol if dtype == F32 else 3e-2), i
    assert rows_rel(lg, want) < tol
    eng = engine_of(model, cache)
    for sizes in ([T], [T - 20] + [1] * 20, [2] * 30 + [1], [7, 33, 2, 16, 3], [1] * T):
        assert rows_rel(steps(eng, "a", toks, sizes), want) < tol, sizes


@pytest.mark.parametrize("name", ["mixed", "odd", "wide"])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_unequal_batches_and_reused_pages_and_slots(name, dtype):
    """Requests of different lengths in one batch, decoded together, against each alone; then the same through pages and slots that were
    freed in another order and still hold the earlier requests' rows and state."""
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 12, dtype, max_tokens=512, max_requests=4, page_size=8)
    eng = engine_of(model, cache)
    lens = {"a": 1, "b": 37, "c": 18, "d": 50}
    n_dec = 14
    toks = {r: tokens_of(cfg, n + n_dec, 40 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: R.forward(P, cfg, t) for r, t in toks.items()}
    for order in (list(lens), ["c", "d", "a", "b"]):
        got = {r: [] for r in order}
        lg = eng.step([{"id": r, "tokens": toks[r][:lens[r]], "want": list(range(lens[r]))} for r in order])
        at = 0
        for r in order:
            got[r].append(lg[at:at + lens[r]])
            at += lens[r]
        live = list(order)
        for k in range(n_dec):
            if k == 5:
                live = live[1:]                      # a shorter request ends earlier
                cache.release(order[0])
            lg = eng.step([{"id": r, "tokens": [toks[r][lens[r] + k]], "want": [0]} for r in live])
            for i, r in enumerate(live):
                got[r].append(lg[i:i + 1])
        for r in order:
            g_ = torch.cat(got[r])
            assert rows_rel(g_, want[r][:g_.shape[0]]) < TOL[dtype], (order, r)
        for r in reversed(live):
            cache.release(r)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_long_decoding_across_windows_and_pages(dtype):
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 14, dtype, page_size=8)
    toks = tokens_of(cfg, 9 + 150, 3)
    want = R.forward(P, cfg, toks)
    assert rows_rel(steps(engine_of(model, cache), "a", toks, [9] + [1] * 150), want) < TOL[dtype]


def test_a_far_token_and_a_kept_token_matter_in_the_model():
    """Changing ONE token far outside every window must still reach the last logits through the kept first tokens (and must not
    when the changed token is neither kept nor within reach), in the framework as in the statement."""
    cfg = R.make_config([R.attention_layer(window=4, keep_first=2, conv=2, mlp=None)])
    model, cache, P = build(cfg, 15, F32, page_size=8)
    eng = engine_of(model, cache)
    T = 60
    base = tokens_of(cfg, T, 1)
    ref0 = R.forward(P, cfg, base)[-1]
    got0 = steps(eng, "a", base, [T - 1, 1])[-1]
    for pos, reaches in ((1, True), (2, False), (T - 6, False), (T - 5, True), (T - 4, True)):
        # (position T - 5 enters through the convolution's two taps: the key at T - 4 reads it)
        alt = list(base)
        alt[pos] = (alt[pos] + 1) % cfg["vocab"]
        ref = R.forward(P, cfg, alt)[-1]
        assert (float((ref - ref0).abs().max()) > 1e-9) == reaches, pos
        got = steps(eng, "b", alt, [T - 1, 1])[-1]
        assert rel(got, ref) < 3e-4
        assert (float((got - got0).abs().max()) > 1e-7) == reaches, pos


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_cache_outgrows_its_first_size(dtype):
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 17, dtype, max_tokens=16, max_requests=1, page_size=8)
    toks = {"a": tokens_of(cfg, 70, 1), "b": tokens_of(cfg, 33, 2)}
    eng = engine_of(model, cache)
    lg = eng.step([{"id": r, "tokens": t[:-4], "want": [len(t) - 5]} for r, t in toks.items()])
    rows = {r: [lg[i:i + 1]] for i, r in enumerate(toks)}
    for k in range(4, 0, -1):
        lg = eng.step([{"id": r, "tokens": [t[-k]], "want": [0]} for r, t in toks.items()])
        for i, r in enumerate(toks):
            rows[r].append(lg[i:i + 1])
    for r, t in toks.items():
        assert rows_rel(torch.cat(rows[r]), R.forward(P, cfg, t)[-5:]) < TOL[dtype]


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_greedy_generation_through_both_loops(dtype):
    """util.generate.prefill_and_generate (one request, chunked prefill, the decode step replayed from a captured HIP graph) and
    BatchEngine.generate (a batch of unequal prompts) against the plain statement's greedy continuation."""
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_vigodra import vigodra_layer_specs
    from ktransformers_amd.util.generate import prefill_and_generate
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 16, dtype, page_size=16)
    prompts = {"p": tokens_of(cfg, 19, 7), "q": tokens_of(cfg, 5, 8)}
    n_new = 12
    out = engine_of(model, cache).generate(prompts, max_new_tokens=n_new)
    for rid, prompt in prompts.items():
        assert len(out[rid]) == n_new
        lg = R.forward(P, cfg, prompt + out[rid])
        for k, tok in enumerate(out[rid]):      # teacher-forced on the framework's own tokens: the argmax wherever its margin is clear
            row = lg[len(prompt) - 1 + k]
            top2 = row.topk(2).values
            if float(top2[0] - top2[1]) > (1e-3 if dtype == F32 else 0.25):
                assert tok == int(row.argmax()), (rid, k)
    for use_graph in (False, True):
        c1 = KHybridCache(vigodra_layer_specs(model.config), 256, max_requests=1, page_size=16, dtype=dtype, device=DEV)
        ids = torch.tensor([prompts["p"]], dtype=torch.int64, device=DEV)
        toks = prefill_and_generate(model, ids, c1, max_new_tokens=n_new, use_cuda_graph=use_graph, chunk_size=8).tolist()
        assert toks == out["p"], (use_graph, toks, out["p"])


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps of a batch replayed from a captured HIP graph, with eager work (another request's prompt) and a change of the
    batch between replays: every replay against the eager engine's logits and against the plain statement."""
    cfg = CONFIGS["wide"]()
    model, cache, P = build(cfg, 21, dtype, page_size=16)
    _, cache2, _ = build(cfg, 21, dtype, page_size=16)
    eager, graphed = engine_of(model, cache2), engine_of(model, cache, use_graph=True)
    reqs = {"a": tokens_of(cfg, 30, 1), "b": tokens_of(cfg, 9, 2)}
    cont = {r: tokens_of(cfg, 12, 30 + i) for i, r in enumerate(reqs)}
    ref = {r: R.forward(P, cfg, reqs[r] + cont[r]) for r in reqs}
    for eng in (eager, graphed):
        eng.step([{"id": r, "tokens": t, "want": []} for r, t in reqs.items()])
    live = list(reqs)
    for k in range(12):
        if k == 4:      # eager work between replays: a third request's prompt through the same cache
            for eng in (eager, graphed):
                eng.step([{"id": "z", "tokens": tokens_of(cfg, 21, 77), "want": [20]}], ["z"])
        if k == 8:
            live = ["a"]
        entries = [{"id": r, "tokens": [cont[r][k]], "want": [0]} for r in live]
        e, g_ = eager.step(entries), graphed.step(entries)
        assert rows_rel(g_, e) < (1e-6 if dtype == F32 else 1e-2), k
        for i, r in enumerate(live):
            assert rows_rel(g_[i:i + 1], ref[r][len(reqs[r]) + k:len(reqs[r]) + k + 1]) < TOL[dtype], (k, r)
