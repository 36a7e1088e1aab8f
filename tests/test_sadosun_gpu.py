"""Sadosun on the GPU against the plain CPU statement of the design (oracle/sadosun_ref.py, fp64): every mechanism alone through its
kernels and operator, then the model through the framework's registry, cache manager, step function and generation loops — whole
prompts, token-by-token decoding, portions, unequal batches, reused pages and slots, keys at the window's edge and at page borders,
odd sizes.  Small random configurations; fp32 runs are held to rounding, bf16 runs to bf16 rounding."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import sadosun_ref as R

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


def rows_close(got, ref, dtype, f32_tol=None):
    """Logit rows against the plain statement.  fp32: every row to rounding.  bf16: rows to bf16 rounding — except that a router score
    within rounding of the next expert's may pick the other expert for a token, which moves that row (and, through the recurrent
    layers and the convolutions, some later ones) by more: the median row is held to the bf16 bound, at most one row in five may exceed
    twice that, none by a gross amount."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    e = (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
    if dtype == F32:
        return float(e.max()) < (f32_tol or TOL[F32])
    return float(e.max()) < 0.5 and float(e.median()) < TOL[BF16] and int((e > 0.12).sum()) <= max(1, e.numel() // 5)


def build(cfg, seed, dtype, max_tokens=2048, max_requests=8, page_size=16, P=None):
    from ktransformers_amd.models import load_model
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_sadosun import sadosun_layer_specs
    from ktransformers_amd.util.loader import DictLoader
    P = R.random_checkpoint(cfg, seed) if P is None else P
    model, config, _ = load_model(cfg, dtype=dtype, device=DEV, loader=DictLoader(P))
    cache = KHybridCache(sadosun_layer_specs(config), max_tokens, max_requests=max_requests, page_size=page_size, dtype=dtype, device=DEV)
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


CONFIGS = {
    # attention and scan layers, grouped heads, a window shorter than the prompts, identity experts, a layer without feed-forward
    "mixed": lambda: R.make_config([R.attention_layer(mlp=R.moe_mlp()), R.scan_layer(mlp=R.moe_mlp(experts=3, top=3, identity=3)),
                                    R.attention_layer(heads=2, kv_heads=2, window=7, rot_dims=8, mlp=None), R.scan_layer(state=20, mlp=R.moe_mlp())]),
    # nothing a multiple of anything: odd width and vocab, 3 heads over 1 key head, vdim != dim, partial rotation, 2 taps, top = 1,
    # no identity expert, a state that is no power of two, dt_rank 1, an embedding scale that is no power of two
    "odd": lambda: R.make_config([R.attention_layer(heads=3, kv_heads=1, dim=10, vdim=6, window=5, rot_dims=4, base=77.0, scale=0.7,
                                                    mlp=R.moe_mlp(experts=3, top=1, identity=0, ff=7)),
                                  R.scan_layer(inner=21, state=5, dt_rank=1, conv=2, mlp=None),
                                  R.attention_layer(heads=6, kv_heads=3, dim=12, vdim=80, window=None, mlp=R.moe_mlp(experts=2, top=2, identity=1, ff=21))],
                                 width=40, vocab=53, eps=1e-3, taps=2, side=3, scale=2.5),
    # sizes the matrix-core attention takes (bf16): dim 32 / 64, vdim 32 / 64, several query heads per key head; every output chosen
    "wide": lambda: R.make_config([R.attention_layer(heads=8, kv_heads=2, dim=32, vdim=64, window=24, mlp=R.moe_mlp(experts=4, top=6, identity=2, ff=32)),
                                   R.scan_layer(inner=256, state=16, dt_rank=8, conv=4, mlp=R.moe_mlp(experts=8, top=2, identity=0, ff=64)),
                                   R.attention_layer(heads=4, kv_heads=4, dim=64, vdim=32, window=None, rot_dims=32, mlp=None)],
                                  width=128, vocab=200, taps=4, side=16),
    # what the config may leave out: no input convolution, no side input, no rotation, no window, one tap in the scan's convolution
    "plain": lambda: R.make_config([R.scan_layer(inner=16, state=3, dt_rank=2, conv=1, mlp=R.moe_mlp(experts=8, top=3, identity=1)),
                                    R.attention_layer(heads=1, kv_heads=1, window=1, rot=False, mlp=None),
                                    R.attention_layer(heads=2, kv_heads=1, window=None, rot=False, mlp=R.moe_mlp(experts=1, top=1, identity=4))],
                                   width=24, taps=0, side=0, scale=1.0),
    # sizes that are 1: one tap in the input convolutions, one head, a window of one, one expert, one state entry, a side input of one
    "ones": lambda: R.make_config([R.attention_layer(heads=1, kv_heads=1, dim=2, vdim=2, window=1, rot_dims=2, mlp=R.moe_mlp(experts=1, top=1, identity=0, ff=1)),
                                   R.scan_layer(inner=1, state=1, dt_rank=1, conv=1, mlp=R.moe_mlp(experts=1, top=2, identity=1, ff=3)),
                                   R.attention_layer(heads=2, kv_heads=1, dim=4, vdim=2, window=2, rot_dims=0, mlp=None)],
                                  width=8, vocab=9, taps=1, side=1, scale=1.0),
}


def batch_of(lens, pos0=None, slots=None, page_size=16, pages=None):
    """A ForwardBatch by hand: requests of `lens` new tokens that start at pos0, in slots `slots`, on consecutive pages."""
    from ktransformers_amd.models.custom_cache import ForwardBatch
    B = len(lens)
    pos0 = pos0 or [0] * B
    slots = slots or list(range(B))
    d = {k: [] for k in ("positions", "tok_req", "cache_loc", "page_indices")}
    q_indptr, page_indptr, at_page = [0], [0], 0
    for b, n in enumerate(lens):
        need = (pos0[b] + n + page_size - 1) // page_size
        mine = pages[b] if pages else list(range(at_page, at_page + need))
        at_page += need
        for p in range(pos0[b], pos0[b] + n):
            d["positions"].append(p)
            d["tok_req"].append(b)
            d["cache_loc"].append(mine[p // page_size] * page_size + p % page_size)
        q_indptr.append(q_indptr[-1] + n)
        d["page_indices"].extend(mine)
        page_indptr.append(len(d["page_indices"]))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return ForwardBatch(T=sum(lens), B=B, max_q_len=max(lens), max_kv_len=max(p + n for p, n in zip(pos0, lens)), nsplit=1,
                        q_indptr=i32(q_indptr), pos0=i32(pos0), slot=i32(slots), page_indptr=i32(page_indptr),
                        **{k: i32(v) for k, v in d.items()})


# ---- mechanisms alone ----------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("W,taps", [(48, 3), (37, 2), (300, 4), (5000, 3), (64, 0), (40, 1), (24, 9), (16, 10)])
def test_scalar_norm_residual_update_and_input_convolution(W, taps):
    from ktransformers_amd._native_swa import input_conv, resid_norm
    g = torch.Generator().manual_seed(W)
    eps, gw = 1e-3, torch.tensor([1.3])
    w = torch.randn(W, max(taps, 1), generator=g) * 0.5
    lens = [7, 1, 12]
    seqs = [torch.randn(n, W, generator=g) * 3 + 0.5 for n in lens]
    ys = [torch.randn(n, W, generator=g) for n in lens]
    want = [R.input_conv(R.scalar_norm((s + y).double(), gw.double(), eps), w.double()) if taps else R.scalar_norm((s + y).double(), gw.double(), eps)
            for s, y in zip(seqs, ys)]
    # whole sequences in one batch, then the same cut in two steps with the state carried in slots that held garbage
    for cuts in ([0], [0, 3], [0, 1, 2], [0, 1, 2, 3, 4, 5]):
        state = torch.full((5, max(taps - 1, 1), W), 7.0, device=DEV)
        slots = [4, 0, 2]
        got = [[] for _ in lens]
        bounds = [[min(c, n) for c in cuts] + [n] for n in lens]
        for k in range(len(cuts)):
            live = [b for b in range(3) if bounds[b][k + 1] > bounds[b][k]]
            if not live:
                continue
            fb = batch_of([bounds[b][k + 1] - bounds[b][k] for b in live], pos0=[bounds[b][k] for b in live], slots=[slots[b] for b in live])
            x = torch.cat([seqs[b][bounds[b][k]:bounds[b][k + 1]] for b in live]).to(DEV)
            y = torch.cat([ys[b][bounds[b][k]:bounds[b][k + 1]] for b in live]).to(DEV)
            if taps == 1 or (1 < taps <= 9 and fb.max_q_len == 1):    # no neighbours, or one token per request: the norm's own launch
                h = resid_norm(x, y=y, norm=(gw.to(DEV), eps), conv=(w.to(DEV), fb, state if taps > 1 else None))
            elif taps > 1:
                hx = resid_norm(x, y=y, norm=(gw.to(DEV), eps), halo=(taps - 1, fb, state))
                h = input_conv(hx, w.to(DEV), fb, state)
            else:
                h = resid_norm(x, y=y, norm=(gw.to(DEV), eps))
            assert rel(x, torch.cat([(seqs[b] + ys[b])[bounds[b][k]:bounds[b][k + 1]] for b in live])) < 1e-6      # x updated in place
            at = 0
            for b in live:
                n = bounds[b][k + 1] - bounds[b][k]
                got[b].append(h[at:at + n])
                at += n
        for b in range(3):
            assert rel(torch.cat(got[b]), want[b]) < 2e-6, (cuts, b)


def test_residual_update_terms():
    """y with its own unit-RMS norm and weight, the mixture's gathered rows with identity choices, a row gather, bf16 outputs."""
    from ktransformers_amd._native_swa import resid_norm
    g = torch.Generator().manual_seed(5)
    d = lambda t: t.to(DEV)
    for W in (40, 257):
        T, top, n_real = 6, 3, 4
        x, y = torch.randn(T, W, generator=g) * 2, torch.randn(T, W, generator=g) * 5
        yw, gw, eps = torch.randn(W, generator=g), torch.tensor([0.8]), 1e-2
        xr = d(x.clone())
        h = resid_norm(xr, y=d(y), y_norm=(d(yw), eps), norm=(d(gw), eps), out_dtype=BF16)
        ref = x.double() + R.unit_rms(y.double(), eps) * yw.double()
        assert rel(xr, ref) < 1e-6 and rel(h, R.scalar_norm(ref, gw.double(), eps)) < 4e-3
        er = torch.randn(T * top, W, generator=g)
        pos = torch.randperm(T * top, generator=g).int()
        idx = torch.randint(0, n_real + 2, (T, top), generator=g).int()
        idx[0], idx[1] = n_real, 0                      # a token with identity choices only, one with real ones only
        tw = torch.rand(T, top, generator=g)
        for hd in (F32, BF16):
            h_in = (torch.randn(T, W, generator=g)).to(hd)
            er_dev = d(er.clone())
            er_dev[pos.long()[(idx >= n_real).reshape(-1)]] = float("nan")       # rows of identity choices are never read
            xr = d(x.clone())
            out = resid_norm(xr, moe=(er_dev, d(pos), d(idx), d(tw), n_real, d(h_in)))
            assert out is None
            pick = torch.where((idx < n_real).unsqueeze(-1), er.double()[pos.long()].view(T, top, W), h_in.double().unsqueeze(1).expand(T, top, W))
            assert rel(xr, x.double() + (pick * tw.double().unsqueeze(-1)).sum(1)) < 1e-6
        rows = torch.tensor([5, 0, 0, 2], dtype=torch.int32)
        assert rel(resid_norm(d(x), norm=(d(gw), eps), rows=d(rows)), R.scalar_norm(x.double(), gw.double(), eps)[rows.long()]) < 1e-6


def attn_op(c, W, dtype, P, page_size=16, tokens=512, slots=4):
    """The injected attention operator alone, with a cache of its own."""
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_sadosun import SadosunAttention
    from ktransformers_amd.operators.window_attention import KWindowGQAttention
    from ktransformers_amd.util.loader import DictLoader
    config = SimpleNamespace(width=W, eps=1e-5, compute_dtype=dtype)
    op = KWindowGQAttention("mix", DictLoader(P), config, SadosunAttention(config, c), generate_device=DEV, prefill_device=DEV)
    op.load()
    cache = KHybridCache([op.state_spec()], tokens, max_requests=slots, page_size=page_size, dtype=dtype, device=DEV)
    return op, cache


def attn_weights(c, W, g, boost=1.0):
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    m = lambda o, i, s: (torch.randn(o, i, generator=g) * s).to(BF16)
    return {"mix.q": m(H * D, W, boost / math.sqrt(W)), "mix.k": m(G * D, W, boost / math.sqrt(W)), "mix.v": m(G * V, W, 1 / math.sqrt(W)),
            "mix.o": m(W, H * V, 1 / math.sqrt(H * V))}


ATTN_SIZES = [  # heads, kv_heads, dim, vdim, window, rot_dims (None: all of dim; 0: values turn, q and k do not; -1: no rotation at all)
    (4, 2, 16, 16, 12, None), (2, 1, 16, 8, 9, 0), (2, 2, 32, 32, 9, 0), (3, 1, 10, 6, 5, 4), (6, 3, 12, 80, None, None), (1, 1, 16, 16, 1, None), (2, 1, 24, 8, 9, -1),
    (8, 2, 32, 64, 24, None), (4, 4, 64, 32, None, 32), (16, 1, 32, 32, 40, 16), (2, 2, 96, 96, 20, None), (4, 1, 128, 128, 33, 64),
    (2, 1, 256, 256, 17, None)]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H,G,D,V,window,rot_dims", ATTN_SIZES)
def test_window_attention_whole_portions_and_kernels(dtype, H, G, D, V, window, rot_dims):
    from ktransformers_amd._native_swa import swa_mfma_eligible
    W, T = 48, 75
    g = torch.Generator().manual_seed(H * 100 + D)
    c = R.attention_layer(heads=H, kv_heads=G, dim=D, vdim=V, window=window, rot_dims=None if rot_dims == -1 else rot_dims, base=500.0,
                          rot=rot_dims != -1)["mixer"]
    P = attn_weights(c, W, g, boost=2.0)
    h = (torch.randn(T, W, generator=g)).to(dtype)
    ref = R.attention_mixer(R.as_double(P), "mix.", c, h.double(), 1e-5)
    op, cache = attn_op(c, W, dtype, P)
    tol = 2e-5 if dtype == F32 else 3e-2
    kernels = [True, False] if dtype == BF16 and swa_mfma_eligible(op._config(cache)) else [False]
    for mfma in kernels:
        op.USE_MATRIX_CORES = mfma
        for sizes, split in (([T], 64), ([1] * T, 64), ([2] * 37 + [1], 64), ([5, 30, 17, 23], 4), ([T], 4)):
            op.KEYS_PER_SPLIT = split           # small key ranges: several workgroups share a token's keys and are merged
            cache.admit("a")
            got, at = [], 0
            for n in sizes:
                got.append(op(h[at:at + n].to(DEV), cache.plan([("a", n)]), cache, 0))
                at += n
            cache.release("a")
            assert rel(torch.cat(got), ref) < tol, (mfma, sizes, split)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("D", [8, 32])
@pytest.mark.parametrize("window,query,back", [(16, 40, 15), (16, 40, 16), (16, 15, 15), (16, 16, 16), (8, 8, 7), (8, 8, 8), (33, 64, 32),
                                               (33, 64, 33), (40, 200, 39), (40, 200, 40), (0, 300, 299), (0, 129, 128)])
def test_one_key_at_the_window_edge_stands_out(dtype, window, query, back, D):
    """One value row is large; the query's score for that key is large.  Just inside the window (or far back without one) it dominates
    the output, just outside it must not be seen — in a whole prompt, decoded token by token, and in portions of two (page size 16:
    positions 15 / 16, 32 / 33, 128 cross page borders)."""
    W, H, G, V = 16, 2, 1, D
    g = torch.Generator().manual_seed(window * 7 + back)
    c = R.attention_layer(heads=H, kv_heads=G, dim=D, vdim=V, window=window or None, rot=False, scale=8.0 / D)["mixer"]
    P = attn_weights(c, W, g)
    T = query + 3
    h = torch.randn(T, W, generator=g) * 0.3
    key_pos = query - back
    # make the key at key_pos and the query at `query` point the same way, strongly; its value large
    direction = torch.randn(W, generator=g)
    h[key_pos], h[query] = direction * 3.0, direction * 1.0
    P["mix.k"] = P["mix.q"][:D].clone()
    h = h.to(dtype)
    ref = R.attention_mixer(R.as_double(P), "mix.", c, h.double(), 1e-5)
    seen = not window or back < window
    plain = ref[query].norm()
    # the statement itself tells the two cases apart (the test's premise)
    other = R.attention_mixer(R.as_double(P), "mix.", c, torch.cat([h[:key_pos], h[key_pos:key_pos + 1] * 0, h[key_pos + 1:]]).double(), 1e-5)
    assert ((ref[query] - other[query]).norm() > 0.2 * plain) == seen
    op, cache = attn_op(c, W, dtype, P)
    tol = 2e-5 if dtype == F32 else 3e-2
    for sizes in ([T], [query - 1] + [1] * 4, [1] * T, [2] * (T // 2) + [1] * (T % 2)):
        cache.admit("a")
        got, at = [], 0
        for n in sizes:
            got.append(op(h[at:at + n].to(DEV), cache.plan([("a", n)]), cache, 0))
            at += n
        cache.release("a")
        assert rel(torch.cat(got)[query - 2:query + 3], ref[query - 2:query + 3]) < tol, sizes


def scan_op(c, W, dtype, P, slots=4):
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_sadosun import SadosunScanMixer
    from ktransformers_amd.operators.selective_scan import KSelectiveScanMixer
    from ktransformers_amd.util.loader import DictLoader
    config = SimpleNamespace(width=W, eps=1e-5, compute_dtype=dtype)
    op = KSelectiveScanMixer("mix", DictLoader(P), config, SadosunScanMixer(config, c), generate_device=DEV, prefill_device=DEV)
    op.load()
    cache = KHybridCache([op.state_spec()], 64, max_requests=slots, dtype=dtype, device=DEV)
    for t in cache.state_tensors():
        t.fill_(3.0)             # a sequence that starts at position 0 starts from zero whatever its slot holds
    return op, cache


def scan_weights(c, W, g):
    I, N, Rk, K = c["inner"], c["state"], c["dt_rank"], c["conv"]
    m = lambda o, i, s: (torch.randn(o, i, generator=g) * s).to(BF16)
    v = lambda n, mean, s: (mean + torch.randn(n, generator=g) * s).to(BF16)
    return {"mix.in": m(2 * I, W, 1 / math.sqrt(W)), "mix.conv": m(I, K, 0.5), "mix.conv.b": v(I, 0.0, 0.1), "mix.x": m(Rk + 2 * N, I, 1 / math.sqrt(I)),
            "mix.dt": m(I, Rk, 1 / math.sqrt(Rk)), "mix.dt.b": v(I, -1.0, 1.0), "mix.A_log": m(I, N, 0.7), "mix.D": v(I, 1.0, 0.3),
            "mix.o": m(W, I, 1 / math.sqrt(I))}


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("I,N,Rk,K", [(48, 8, 4, 3), (21, 5, 1, 2), (64, 16, 8, 4), (130, 33, 3, 4), (300, 70, 5, 1), (16, 130, 2, 5), (256, 32, 16, 4)])
def test_selective_scan_whole_portions_and_state_carry(dtype, I, N, Rk, K):
    W, T = 40, 45
    g = torch.Generator().manual_seed(I + N)
    c = R.scan_layer(inner=I, state=N, dt_rank=Rk, conv=K)["mixer"]
    P = scan_weights(c, W, g)
    h = torch.randn(T, W, generator=g).to(dtype)
    ref = R.mamba_mixer(R.as_double(P), "mix.", c, h.double())
    op, cache = scan_op(c, W, dtype, P)
    tol = 2e-5 if dtype == F32 else 3e-2
    for sizes in ([T], [1] * T, [2] * 22 + [1], [3, 1, 20, 2, 19], [44, 1]):
        cache.admit("a"), cache.admit("b")        # two requests side by side: b runs the same tokens shifted by one step
        got, at = [], 0
        for n in sizes:
            got.append(op(h[at:at + n].to(DEV), cache.plan([("a", n)]), cache, 0))
            at += n
        cache.release("b"), cache.release("a")
        assert rel(torch.cat(got), ref) < tol, sizes
    # a batch of unequal requests equals each alone
    lens = [T, 7, 1, 20]
    for r, n in enumerate(lens):
        cache.admit(r)
    out = op(torch.cat([h[:n] for n in lens]).to(DEV), cache.plan([(r, n) for r, n in enumerate(lens)]), cache, 0)
    at = 0
    for n in lens:
        assert rel(out[at:at + n], ref[:n]) < tol, n
        at += n


def test_selective_scan_remembers_far_tokens():
    """A channel with a slow decay keeps what token 3 wrote for hundreds of steps, across portions and decode steps."""
    W, T, I, N = 16, 400, 8, 4
    g = torch.Generator().manual_seed(9)
    c = R.scan_layer(inner=I, state=N, dt_rank=2, conv=2)["mixer"]
    P = scan_weights(c, W, g)
    P["mix.A_log"] = torch.full((I, N), -9.0).to(BF16)          # A = -e^-9: the state hardly decays
    h = torch.randn(T, W, generator=g) * 0.05
    h[3] = torch.randn(W, generator=g) * 6.0
    ref = R.mamba_mixer(R.as_double(P), "mix.", c, h.double())
    quiet = R.mamba_mixer(R.as_double(P), "mix.", c, torch.cat([h[:3], h[3:4] * 0, h[4:]]).double())
    assert (ref[-1] - quiet[-1]).norm() > 0.5 * ref[-1].norm()    # the premise: the last token's output still rests on token 3
    op, cache = scan_op(c, W, F32, P)
    for sizes in ([T], [10] + [1] * (T - 10), [64] * 6 + [16]):
        cache.admit("a")
        got, at = [], 0
        for n in sizes:
            got.append(op(h[at:at + n].to(DEV), cache.plan([("a", n)]), cache, 0))
            at += n
        cache.release("a")
        assert rel(torch.cat(got)[-20:], ref[-20:]) < 1e-4, sizes[:3]


@pytest.mark.parametrize("E,top,T", [(6, 2, 50), (3, 1, 7), (4, 4, 9), (70, 5, 300), (16, 3, 1), (130, 130, 5)])
def test_softmax_router(E, top, T):
    from ktransformers_amd._native_swa import softmax_route
    g = torch.Generator().manual_seed(E)
    z = torch.randn(T, E + 3, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.1
    P = {"router": torch.eye(E).double(), "correction": corr.double()}
    for use_corr in (True, False):
        idx, w = softmax_route(z.to(DEV)[:, :E], top, 1e-20, corr.to(DEV) if use_corr else None)       # (a column slice: strided rows)
        Pr = P if use_corr else {"router": P["router"]}
        ridx, rw = R.route(Pr, "", {"router": {"top": top}}, z[:, :E].double())
        assert torch.equal(idx.cpu().long().sort(dim=1).values, ridx.sort(dim=1).values)
        order = idx.cpu().long().argsort(dim=1), ridx.argsort(dim=1)
        assert rel(torch.gather(w.cpu(), 1, order[0]), torch.gather(rw, 1, order[1])) < 1e-6
    if T <= 64:      # small steps route and sort in one launch: the same choices, and a sort that puts every pair into its expert's rows
        from ktransformers_amd._native_hyb import moe_plan
        from ktransformers_amd._native_swa import softmax_route_plan
        zc = z.to(DEV)[:, :E].contiguous()
        idx1, w1 = softmax_route(zc, top, 1e-20, corr.to(DEV))
        idx2, w2, plan = softmax_route_plan(zc, top, 1e-20, corr.to(DEV))
        assert torch.equal(idx1, idx2) and torch.equal(w1, w2)
        ref_plan = moe_plan(idx1, E)
        assert torch.equal(plan.group_off, ref_plan.group_off) and int(plan.num_tiles) == int(ref_plan.num_tiles)
        nt = int(plan.num_tiles)
        assert torch.equal(plan.tile_group[:nt], ref_plan.tile_group[:nt]) and torch.equal(plan.tile_row0[:nt], ref_plan.tile_row0[:nt])
        flat, pos = idx2.reshape(-1).long(), plan.pair_pos.long()
        assert sorted(pos.tolist()) == list(range(T * top))
        assert torch.equal(plan.sorted_group.long()[pos], flat) and torch.equal(plan.sorted_tok.long()[pos], torch.arange(T * top, device=DEV) // top)
    # the correction changes the choice, not the weights: a large one on output 0 forces it in, its weight stays its softmax share
    big = torch.zeros(E)
    big[0] = 10.0
    idx, w = softmax_route(z.to(DEV)[:, :E].contiguous(), top, 1e-20, big.to(DEV))
    assert bool((idx == 0).any(dim=1).all())
    s = torch.softmax(z[:, :E].double(), dim=-1)
    assert rel(w.cpu().sum(1), torch.ones(T)) < 1e-6
    k0 = (idx.cpu() == 0).long().argmax(dim=1)
    chosen = torch.gather(s, 1, idx.cpu().long())
    assert rel(torch.gather(w.cpu(), 1, k0.view(-1, 1)), (s[:, 0] / chosen.sum(1)).view(-1, 1)) < 1e-6


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("E,ID,top,F,T", [(5, 2, 2, 24, 50), (3, 0, 1, 7, 9), (4, 2, 6, 32, 130), (16, 1, 3, 40, 1), (2, 1, 2, 136, 400),
                                          (1, 4, 1, 16, 20), (8, 0, 2, 64, 3), (12, 3, 11, 16, 30), (20, 0, 17, 8, 2)])
def test_mixture_with_identity_experts(dtype, E, ID, top, F, T):
    """The operator's pieces, joined by the residual update, against the plain mixture: streaming products (few pairs), 64-row tiles
    and 128-row tiles (many pairs per expert), tokens whose choices are all identity experts."""
    from ktransformers_amd._native_swa import resid_norm
    from ktransformers_amd.models.modeling_sadosun import SadosunMoE
    from ktransformers_amd.operators.softmax_moe import KSoftmaxRoutedMoE
    from ktransformers_amd.util.loader import DictLoader
    W = 40
    g = torch.Generator().manual_seed(E * 10 + top)
    c = R.moe_mlp(experts=E, top=top, identity=ID, ff=F)
    m = lambda o, i, s: (torch.randn(o, i, generator=g) * s).to(BF16)
    P = {"mlp.router": m(E + ID, W, 3 / math.sqrt(W)), "mlp.correction": (torch.randn(E + ID, generator=g) * 0.05).to(BF16)}
    for e in range(E):
        P[f"mlp.e{e}.up"], P[f"mlp.e{e}.down"] = m(F, W, 1 / math.sqrt(W)), m(W, F, 1 / math.sqrt(F))
    config = SimpleNamespace(width=W, eps=1e-5, compute_dtype=dtype)
    op = KSoftmaxRoutedMoE("mlp", DictLoader(P), config, SadosunMoE(config, c), generate_device=DEV, prefill_device=DEV)
    op.load()
    h = torch.randn(T, W, generator=g).to(dtype)
    x = torch.randn(T, W, generator=g)
    xr = x.clone().to(DEV)
    resid_norm(xr, moe=op(h.to(DEV)))
    ref = x.double() + R.moe_ff(R.as_double(P), "mlp.", c, h.double())
    got, ref = xr.double().cpu() - x.double(), ref - x.double()
    e = (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
    if dtype == F32:
        assert float(e.max()) < 2e-5
    else:        # a near-tie in the router may fall the other way for a few tokens
        assert float(e.median()) < 2e-2 and int((e > 6e-2).sum()) <= max(1, T // 10)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_token_side_input(dtype):
    from ktransformers_amd._native_swa import resid_norm
    from ktransformers_amd.models.modeling_sadosun import SadosunSideInput
    from ktransformers_amd.operators.embedding import KTokenSideInput
    from ktransformers_amd.util.loader import DictLoader
    g = torch.Generator().manual_seed(2)
    for W, dim, layers, li, T in ((40, 6, 3, 1, 17), (128, 16, 2, 0, 70), (24, 1, 4, 3, 5)):
        m = lambda o, i, s: (torch.randn(o, i, generator=g) * s).to(BF16)
        P = {"side.gate": m(dim, W, 1 / math.sqrt(W)), "side.proj": m(W, dim, 1.0), "side.norm": (0.7 + torch.randn(W, generator=g) * 0.2).to(BF16)}
        table = m(31, dim * layers, 1.0)
        config = SimpleNamespace(width=W, eps=1e-4, compute_dtype=dtype, side_dim=dim)
        op = KTokenSideInput("side", DictLoader(P), config, SadosunSideInput(config, li), generate_device=DEV, prefill_device=DEV)
        op.load()
        toks = torch.randint(0, 31, (T,), generator=g)
        x = torch.randn(T, W, generator=g) * 2
        xr = x.clone().to(DEV)
        y = op(xr, toks.int().to(DEV), table.to(dtype).to(DEV))
        resid_norm(xr, y=y, y_norm=op.y_norm)
        ref = R.side_input(R.as_double(P), "side.", x.double(), table.double()[toks][:, li * dim:(li + 1) * dim], 1e-4)
        assert rel(xr.double().cpu() - x.double(), ref) < (2e-5 if dtype == F32 else 3e-2), (W, dim)


# ---- the model through the framework -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(dtype, name):
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 11, dtype)
    toks = tokens_of(cfg, 50, 1)
    ref, ref_layers = R.forward(P, cfg, toks, return_layers=True)
    cache.admit("a")
    fb = cache.plan([("a", len(toks))])
    logits, layers = model(torch.tensor(toks, dtype=torch.int32, device=DEV), None, cache, batch=fb, return_layers=True)
    assert layers.shape == ref_layers.shape
    for li in range(ref_layers.shape[0]):
        assert rel(layers[li], ref_layers[li]) < TOL[dtype], f"layer {li}"
    assert rows_close(logits, ref, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("name", ["mixed", "odd", "wide", "ones"])
def test_prefill_equals_token_by_token_and_portions(dtype, name):
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 12, dtype, page_size=8)
    eng = engine_of(model, cache)
    toks = tokens_of(cfg, 41, 2)
    ref = R.forward(P, cfg, toks)
    whole = steps(eng, "w", toks, [41])
    assert rows_close(whole, ref, dtype)
    for sizes in ([1] * 41, [2] * 20 + [1], [3, 5, 8, 9, 16], [39, 2], [7] + [1] * 34):
        got = steps(eng, "p", toks, sizes)
        assert rows_close(got, ref, dtype), sizes
        assert rows_close(got, whole, dtype, f32_tol=2e-5), sizes      # cutting the prompt changes rounding only
    assert not cache.requests and len(cache.free_pages) == cache.num_pages


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_unequal_batch_equals_each_alone_and_reuses_pages_and_slots(dtype):
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 13, dtype, max_tokens=400, max_requests=3, page_size=8)
    eng = engine_of(model, cache)
    reqs = {"a": tokens_of(cfg, 1, 3), "b": tokens_of(cfg, 37, 4), "c": tokens_of(cfg, 90, 5)}
    tail = 6
    alone = {rid: R.forward(P, cfg, toks + tokens_of(cfg, tail, 50 + len(toks))) for rid, toks in reqs.items()}
    for round_ in range(3):       # every round takes the pages and slots the previous one gave back, in another order
        order = list(reqs)[round_:] + list(reqs)[:round_]
        lg = eng.step([{"id": r, "tokens": reqs[r], "want": [len(reqs[r]) - 1]} for r in order])
        got, ref = [lg], [torch.stack([alone[r][len(reqs[r]) - 1] for r in order])]
        live = list(order)
        for step in range(tail):
            ext = {r: tokens_of(cfg, tail, 50 + len(reqs[r]))[step] for r in live}
            ending = [r for r in live if (r == "a" and step == 1) or step == tail - 1]       # the short request leaves early
            lg = eng.step([{"id": r, "tokens": [ext[r]], "want": [0]} for r in live], ending)
            got.append(lg)
            ref.append(torch.stack([alone[r][len(reqs[r]) + step] for r in live]))
            live = [r for r in live if r not in ending]
        assert rows_close(torch.cat(got), torch.cat(ref), dtype), round_
        assert not cache.requests


def test_long_decoding_past_windows_and_pages():
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 14, F32, page_size=16)
    eng = engine_of(model, cache)
    toks = tokens_of(cfg, 150, 6)
    ref = R.forward(P, cfg, toks)
    got = [eng.step([{"id": "d", "tokens": toks[:10], "want": [9]}])]
    for t in range(10, len(toks)):
        got.append(eng.step([{"id": "d", "tokens": [toks[t]], "want": [0]}]))
    assert rows_rel(torch.cat(got), ref[9:]) < TOL[F32]


def test_cache_grows_beyond_its_first_size():
    cfg = CONFIGS["mixed"]()
    model, cache, P = build(cfg, 15, F32, max_tokens=32, max_requests=1, page_size=8)
    eng = engine_of(model, cache)
    reqs = {k: tokens_of(cfg, 30 + 7 * k, k) for k in range(4)}          # more requests and tokens than the cache was made for
    lg = eng.step([{"id": k, "tokens": t, "want": [len(t) - 1]} for k, t in reqs.items()])
    for i, (k, t) in enumerate(reqs.items()):
        assert rows_rel(lg[i:i + 1], R.forward(P, cfg, t)[-1:]) < TOL[F32]
    lg = eng.step([{"id": k, "tokens": [5], "want": [0]} for k in reqs])  # and the state survived the re-allocation
    for i, (k, t) in enumerate(reqs.items()):
        assert rows_rel(lg[i:i + 1], R.forward(P, cfg, t + [5])[-1:]) < TOL[F32]


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_greedy_generation_through_both_loops(dtype):
    """util.generate.prefill_and_generate (one request, chunked prefill, the decode step replayed from a captured HIP graph) and
    BatchEngine.generate (a batch of unequal prompts) against the plain statement's greedy continuation."""
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_sadosun import sadosun_layer_specs
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
        c1 = KHybridCache(sadosun_layer_specs(model.config), 256, max_requests=1, page_size=16, dtype=dtype, device=DEV)
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
    live, got, want = list(reqs), [], []
    for k in range(12):
        entries = [{"id": r, "tokens": [cont[r][k]], "want": [0]} for r in live]
        end = ["b"] if k == 6 else []
        le, lg = eager.step(entries, end), graphed.step(entries, end)
        assert rows_rel(lg, le) < (1e-5 if dtype == F32 else 2e-2), k
        got.append(lg)
        want.append(torch.stack([ref[r][len(reqs[r]) + k] for r in live]))
        live = [r for r in live if r not in end]
        if k == 3:      # eager work between two replays
            for eng in (eager, graphed):
                eng.step([{"id": "c", "tokens": tokens_of(cfg, 20, 9), "want": [19]}], ["c"])
    assert rows_close(torch.cat(got), torch.cat(want), dtype)
    assert len(graphed._graphs) >= 2
