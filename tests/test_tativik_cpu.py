"""The sandwich arrangement of the hybrid family (the Tativik design) without a GPU: the reader of
config.json, the weight layout, page accounting, and properties of the plain restatement that the
GPU tests lean on (window edge, sink, routing inside kept groups, cut invariance of the recurrence)."""
import pytest
import torch

from oracle import tativik_ref as R


def _cfg():
    lat = {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "kv_rank": 40, "q_rank": 24, "mask": {"size": 20},
           "rot": {"dims": 4, "base": 1000.0}, "scale": 0.2}
    moe = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 6, "top": 3, "groups": {"count": 3, "keep": 2}}}
    return {"architecture": "Tativik", "width": 96, "vocab": 160, "norm": {"eps": 1e-5, "groups": 3}, "residual_mult": 0.5,
            "layers": [{"type": "latent_attention", "mixer": lat, "mlp": moe},
                       {"type": "general_delta", "mixer": {"heads": 2, "dim": 32}, "mlp": None},
                       {"type": "latent_attention", "mixer": dict(lat, heads=2, kv_from=0), "mlp": moe}]}


def test_config_reader():
    from mi355_decode.config import ModelConfig
    cfg = ModelConfig.from_dict(_cfg())
    spec = cfg.hybrid
    assert cfg.family == "hybrid" and cfg.architecture == "Tativik" and cfg.vocab_size == 160 and cfg.hidden_size == 96
    assert spec.arrangement == "sandwich" and spec.norm_groups == 3 and spec.residual_mult == 0.5
    assert [L.kind for L in spec.layers] == ["latent_attention", "general_delta", "latent_attention"]
    a, b = spec.layers[0].lattn, spec.layers[2].lattn
    assert (a.window, a.rot_dims, a.rot_dim, a.kv_from, b.kv_from, b.heads) == (20, 4, 8, None, 0, 2)
    m = spec.layers[0].moe
    assert (m.experts, m.top, m.groups, m.keep, m.ff) == (6, 3, 3, 2, 40) and spec.layers[1].moe is None
    assert spec.runs() == [(0, None), (1, None), (2, None)]
    bad = _cfg()
    bad["layers"][2]["mixer"]["kv_from"] = 1                  # not a latent attention
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][2]["mixer"]["kv_rank"] = 48                 # another latent size than the layer it reads
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][0]["mlp"]["router"]["top"] = 5              # two kept groups of two experts hold four
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)


def test_weight_layout_and_page_accounting():
    from mi355_decode import weights as W
    from mi355_decode.config import ModelConfig
    d = _cfg()
    cfg = ModelConfig.from_dict(d)
    st = R.random_state(d, seed=1)
    w = W.from_state_dict(cfg, st, torch.float32, "cpu")
    l0, l1, l2 = w.layers
    assert list(l0.seg) == ["dq", "dkv", "g", "rg"] and list(l2.seg) == ["dq", "g", "rg"]
    assert list(l1.seg) == ["r", "k", "v", "g", "a", "w1", "rg"]
    for lw in w.layers:
        assert all(a % 8 == 0 for a, _ in lw.seg.values())
        a, n = lw.seg["rg"]
        assert n == 96 and lw.in_w.shape[0] == a + 96
    a, n = l0.seg["dkv"]
    assert torch.equal(l0.in_w[a:a + n], st["l0.mix.dkv"]) and l2.dkv_norm is None
    assert l0.uk_w.shape == (3, 16, 40) and l0.uv_t.shape == (3, 40, 24)
    assert torch.equal(l0.uv_t[1], st["l0.mix.uv"][24:48].T)
    assert l0.gate_up_w.shape == (6, 80, 96) and torch.equal(l0.gate_up_w[4, 40:], st["l0.mlp.e4.up"])
    assert l0.router_w.dtype == torch.float32 and l1.gate_up_w is None and w.embed_norm.shape == (96,)
    # synthetic weights come under the same names
    assert set(W.hybrid_synthetic_state(cfg, seed=0)) == set(st)
    # a configuration that names neither the query latent's size nor a window: the tensor's shape, no window
    for L in d["layers"]:
        L["mixer"].pop("q_rank", None)
        L["mixer"].pop("mask", None)
    cfg2 = ModelConfig.from_dict(d)
    assert cfg2.hybrid.layers[0].lattn.q_rank == 0 and cfg2.hybrid.layers[0].lattn.window >= 1 << 30
    w2 = W.from_state_dict(cfg2, st, torch.float32, "cpu")
    assert cfg2.hybrid.layers[0].lattn.q_rank == 24 and torch.equal(w2.layers[0].uq_w, l0.uq_w)


def test_restatement_edges_and_cut_invariance():
    g = torch.Generator().manual_seed(0)
    s = torch.randn(12, 12, generator=g)
    sink = torch.tensor(0.3)
    p = R.window_softmax_with_sink(s, 4, sink)
    for i in range(12):
        seen = [j for j in range(12) if p[i, j] > 0]
        assert seen == list(range(max(0, i - 3), i + 1))
        e = torch.exp(s[i, seen])
        assert torch.allclose(p[i, seen], e / (e.sum() + torch.exp(sink)), atol=1e-6)
        assert float(p[i].sum()) < 1.0                       # the sink holds the rest
    # the recurrence over a whole sequence equals the recurrence restarted from a carried state
    T, H, d = 9, 2, 8
    r, k, v = (torch.randn(T, H, d, generator=g) for _ in range(3))
    w, a = torch.rand(T, H, d, generator=g), torch.rand(T, H, d, generator=g)
    whole = R.general_delta_rule(r, k, v, w, a)
    S = torch.zeros(H, d, d)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        S = w[t][:, :, None] * S - (a[t] * u)[:, :, None] * torch.einsum("hi,hij->hj", u, S)[:, None, :] \
            + k[t][:, :, None] * v[t][:, None, :]
        assert torch.allclose(torch.einsum("hij,hi->hj", S, r[t]), whole[t], atol=1e-5)


def test_restatement_routes_inside_the_kept_groups():
    g = torch.Generator().manual_seed(3)
    z = torch.randn(200, 12, generator=g)
    corr = torch.randn(12, generator=g) - 2.0                 # every choice score below zero
    ids, wts = R.route(z, corr, 3, 4, 2)
    choice = torch.sigmoid(z) + corr
    gs = choice.view(200, 4, 3).topk(2, dim=-1).values.sum(-1)
    for t in range(200):
        kept = set(gs[t].topk(2).indices.tolist())
        assert {int(e) // 3 for e in ids[t]} <= kept
        allowed = [e for e in range(12) if e // 3 in kept]
        assert sorted(ids[t].tolist()) == sorted(sorted(allowed, key=lambda e: -float(choice[t, e]))[:3])
        assert torch.allclose(wts[t], torch.sigmoid(z[t, ids[t]]))
