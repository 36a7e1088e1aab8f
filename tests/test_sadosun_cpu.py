"""Host side of the Sadosun family, no GPU: the plain statement's own consistency (causality, the window's edges, the sink, values that
enter relative to the query, the scan carried token by token, identity experts, the choice correction), config reading, the registry,
rule injection on the meta device, and the cache / state manager's key + value caches and convolution slots."""
import os

import pytest
import torch

from oracle import sadosun_ref as R


def test_statement_is_causal_and_the_window_has_the_edges_it_says():
    cfg = R.make_config([R.attention_layer(heads=2, kv_heads=1, window=4)])
    P = R.as_double(R.random_checkpoint(cfg, 1))
    c = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(0)
    h = torch.randn(12, 32, generator=g).double()
    full = R.attention_mixer(P, "l0.mix.", c, h, 1e-5)
    assert torch.allclose(R.attention_mixer(P, "l0.mix.", c, h[:7], 1e-5), full[:7], atol=1e-12)       # later tokens change nothing
    h2 = h.clone()
    h2[5] += 1.0                         # position 5 is seen by 5 .. 8 (window 4) and by nobody else
    moved = (R.attention_mixer(P, "l0.mix.", c, h2, 1e-5) - full).abs().amax(-1) > 1e-9
    assert moved.tolist() == [False] * 5 + [True] * 4 + [False] * 3
    # the sink: a single visible key with score s gets weight e^s / (1 + e^s), never 1
    one = R.attention_mixer(P, "l0.mix.", c, h[:1], 1e-5)
    c0 = dict(c, rot=None)
    v = (h[:1] @ P["l0.mix.v"].T).view(1, 1, 16)
    q = R.unit_rms((h[:1] @ P["l0.mix.q"].T).view(1, 2, 16), 1e-5)
    k = R.unit_rms((h[:1] @ P["l0.mix.k"].T).view(1, 1, 16), 1e-5)
    s = (q * k).sum(-1) * c["scale"]
    want = (torch.sigmoid(s).unsqueeze(-1) * v).reshape(1, 32) @ P["l0.mix.o"].T       # position 0: every rotation is the identity
    assert torch.allclose(one, want, atol=1e-12) and torch.allclose(R.attention_mixer(P, "l0.mix.", c0, h[:1], 1e-5), want, atol=1e-12)


def test_values_enter_relative_to_the_query():
    """Turning values by their position and the result back by the query's = turning each value by (j - i): shifting the whole sequence
    changes nothing when keys and queries are not rotated (rot.dims = 0)."""
    c = R.attention_layer(heads=1, kv_heads=1, dim=4, vdim=6, window=None, rot_dims=0, base=30.0)["mixer"]
    g = torch.Generator().manual_seed(3)
    P = {"q": torch.randn(4, 8, generator=g).double(), "k": torch.randn(4, 8, generator=g).double(),
         "v": torch.randn(6, 8, generator=g).double(), "o": torch.eye(6).double()}
    h = torch.randn(9, 8, generator=g).double()
    full = R.attention_mixer(P, "", c, h, 1e-5)
    # by hand for the last position: sum_j p_j turn(v_j, j - 8)
    T = 9
    q = R.unit_rms(h @ P["q"].T, 1e-5)
    k = R.unit_rms(h @ P["k"].T, 1e-5)
    e = torch.exp((k @ q[8]) * c["scale"])
    p = e / (1 + e.sum())
    v = h @ P["v"].T
    rel = torch.arange(T) - 8
    want = (p.unsqueeze(-1) * R.turn_pairs(v, rel, 30.0, 6)).sum(0)
    assert torch.allclose(full[8], want, atol=1e-12)
    x = torch.arange(6, dtype=torch.float64).view(1, 6) + 1
    y = R.turn_pairs(x, torch.tensor([3]), 100.0, 4)
    assert torch.equal(y[0, 4:], x[0, 4:]) and abs(float(y[0, 0]) - (1 * torch.cos(torch.tensor(3.0)) - 2 * torch.sin(torch.tensor(3.0))).item()) < 1e-7
    assert abs(float(y[0, 3]) - (4 * torch.cos(torch.tensor(0.3, dtype=torch.float64)) + 3 * torch.sin(torch.tensor(0.3, dtype=torch.float64))).item()) < 1e-12


def test_convolutions_and_scan_carry():
    conv = R.causal_conv(torch.tensor([[1.0], [10.0], [100.0]]), torch.tensor([[0.5, 2.0, 3.0]]))
    assert conv[:, 0].tolist() == [3.0, 32.0, 320.5]           # last column = the current token, zeros before the start
    assert R.input_conv(torch.tensor([[1.0], [10.0]]), torch.tensor([[2.0, 3.0]]))[:, 0].tolist() == [4.0, 42.0]
    cfg = R.make_config([R.scan_layer(inner=6, state=3, dt_rank=2, conv=2)], width=8)
    P = R.as_double(R.random_checkpoint(cfg, 2))
    h = torch.randn(7, 8, generator=torch.Generator().manual_seed(0)).double()
    c = cfg["layers"][0]["mixer"]
    full = R.mamba_mixer(P, "l0.mix.", c, h)
    assert torch.allclose(R.mamba_mixer(P, "l0.mix.", c, h[:4]), full[:4], atol=1e-12)
    # one token from an empty state: S = dt x B, y = (dt x B . C + D x) silu(z)
    x, z = (h[:1] @ P["l0.mix.in"].T).split(6, dim=1)
    x = R.silu(x * P["l0.mix.conv"][:, -1] + P["l0.mix.conv.b"])
    low = x @ P["l0.mix.x"].T
    dt = R.softplus(low[:, :2] @ P["l0.mix.dt"].T + P["l0.mix.dt.b"])
    y = dt * x * (low[:, 2:5] * low[:, 5:]).sum() + P["l0.mix.D"] * x
    assert torch.allclose(full[:1], (y * R.silu(z)) @ P["l0.mix.o"].T, atol=1e-12)


def test_identity_experts_and_the_choice_correction():
    c = R.moe_mlp(experts=2, top=2, identity=2, ff=4)
    g = torch.Generator().manual_seed(1)
    P = {"router": torch.randn(4, 8, generator=g).double(), "correction": torch.tensor([0.0, 0.0, 5.0, 5.0]).double()}
    for e in range(2):
        P[f"e{e}.up"], P[f"e{e}.down"] = torch.randn(4, 8, generator=g).double(), torch.randn(8, 4, generator=g).double()
    h = torch.randn(5, 8, generator=g).double()
    idx, w = R.route(P, "", c, h)
    assert sorted(idx[0].tolist()) == [2, 3] and torch.allclose(w.sum(1), torch.ones(5).double())      # the correction decides the choice
    s = torch.softmax(h @ P["router"].T, dim=-1)
    assert torch.allclose(w[0], s[0, idx[0]] / s[0, idx[0]].sum())                                      # and stays out of the weights
    assert torch.allclose(R.moe_ff(P, "", c, h), h, atol=1e-12)                                         # identity experts only: h itself


def test_config_reader_checks_and_registry():
    from ktransformers_amd.models import MODEL_REGISTRY, architecture_of
    from ktransformers_amd.models.modeling_sadosun import make_sadosun_config, sadosun_layer_specs
    raw = R.make_config([R.attention_layer(heads=6, kv_heads=3, dim=10, vdim=8, mlp=R.moe_mlp()), R.scan_layer(inner=20, state=5, conv=4)],
                        taps=3, side=7, scale=2.5)
    cfg = make_sadosun_config(raw)
    assert cfg.num_hidden_layers == 2 and cfg.width == raw["width"] and cfg.eps == raw["norm"]["eps"]
    assert cfg.canon_taps == 3 and cfg.side_dim == 7 and cfg.embed_scale == 2.5
    specs = sadosun_layer_specs(cfg)
    assert specs[0] == {"kv": (3, 10, 8), "pre": [(32, 3), (32, 3)]} and specs[1] == {"ssm": (20, 5), "conv": (20, 4), "pre": [(32, 3), None]}
    bare = make_sadosun_config(R.make_config([R.attention_layer(rot=False, window=None)], taps=0, side=0))
    assert bare.canon_taps == 0 and bare.side_dim == 0 and sadosun_layer_specs(bare)[0]["pre"] == [None, None]
    assert architecture_of(raw) == "Sadosun" and torch.float32 in MODEL_REGISTRY["Sadosun"].dtypes
    for breakit, match in ((lambda c: c["layers"][0].update(type="serial"), "layer type"),
                           (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "multiple"),
                           (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "even"),
                           (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
                           (lambda c: c["layers"][0].update(mlp={"kind": "dense"}), "feed-forward")):
        bad = R.make_config([R.attention_layer(heads=6, kv_heads=3, mlp=R.moe_mlp()), R.scan_layer()])
        breakit(bad)
        with pytest.raises(ValueError, match=match):
            make_sadosun_config(bad)


def test_rules_replace_every_arithmetic_leaf():
    from ktransformers_amd.models import RULES_DIR
    from ktransformers_amd.models.modeling_deepseek import _Leaf
    from ktransformers_amd.models.modeling_sadosun import SadosunForCausalLM, make_sadosun_config
    from ktransformers_amd.optimize.optimize import gen_optimize_config, inject, load_rules
    from ktransformers_amd.util.loader import DictLoader
    raw = R.make_config([R.attention_layer(mlp=R.moe_mlp()), R.scan_layer(mlp=R.moe_mlp(identity=0)), R.attention_layer()])
    cfg = make_sadosun_config(raw)
    with torch.device("meta"):
        model = SadosunForCausalLM(cfg)
    plan = {}
    gen_optimize_config(model, plan, load_rules(os.path.join(RULES_DIR, "Sadosun.yaml")))
    inject(model, plan, cfg, DictLoader(R.random_checkpoint(raw, 0)))
    kinds = {n: type(m).__name__ for n, m in model.named_modules() if type(m).__name__.startswith("K")}
    assert kinds["l0.mix"] == "KWindowGQAttention" and kinds["l1.mix"] == "KSelectiveScanMixer"
    assert kinds["l0.mlp"] == kinds["l1.mlp"] == "KSoftmaxRoutedMoE" and "l2.mlp" not in kinds and model.l2.mlp is None
    assert {"embed", "side", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.canon1", "l1.canon2", "l2.side", "l2.canon1"} <= set(kinds)
    assert "l2.norm2" not in kinds
    left = [n for n, m in model.named_modules() if isinstance(m, _Leaf)]
    assert all(".orig_module" in n for n in left)          # every leaf that is left sits behind its operator
    assert model.l0.mix.sink_score == 0.0 and model.l0.mix.rot_values and model.l0.mlp.identity == 2 and model.l1.mlp.identity == 0


def test_cache_manager_keeps_keys_values_and_convolution_slots():
    from ktransformers_amd.models.custom_cache import KHybridCache
    specs = [{"kv": (2, 4, 6), "pre": [(8, 3), (8, 3)]}, {"ssm": (10, 5), "conv": (10, 4), "pre": [(8, 3), None]}, {"kv": (1, 4, 4), "pre": [None, None]}]
    c = KHybridCache(specs, max_tokens=64, max_requests=2, page_size=8, dtype=torch.float32, device="cpu")
    rows = c.num_pages * 8
    assert c.k_caches[0].shape == (rows, 2, 4) and c.v_caches[0].shape == (rows, 2, 6) and c.k_inv[0] is None and c.v_caches[1] is None
    assert c.S[1].shape == (2, 10, 5) and c.conv[1].shape == (2, 3, 10) and c.S[0] is None
    assert [None if t is None else tuple(t.shape) for t in c.pre_conv[0]] == [(2, 2, 8), (2, 2, 8)] and c.pre_conv[1][1] is None
    assert c.pre_conv[2] == [None, None]
    assert len(c.state_tensors()) == 2 + 3
    c.v_caches[0][0, 0, 0] = 5.0
    c.pre_conv[1][0][1, 1, 3] = 2.0
    c.admit("a"), c.admit("b"), c.admit("x")                 # one request more than the cache was made for: slots grow, contents stay
    c.plan([("x", 200)])
    assert c.S[1].shape[0] == c.max_requests >= 3 and c.pre_conv[1][0].shape[0] == c.max_requests and float(c.pre_conv[1][0][1, 1, 3]) == 2.0
    assert c.v_caches[2].shape[0] == c.num_pages * 8 == c.k_caches[2].shape[0] and float(c.v_caches[0][0, 0, 0]) == 5.0
    with pytest.raises(ValueError):
        KHybridCache([{"ssm": (2, 2), "delta": (1, 2, 2)}], 8, dtype=torch.float32, device="cpu")
    with pytest.raises(ValueError):
        KHybridCache([{"attn": (1, 2), "kv": (1, 2, 2)}], 8, dtype=torch.float32, device="cpu")
