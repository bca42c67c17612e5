"""The Tafisun design of the hybrid family without a GPU: the reader of config.json and its refusals,
the weight layout, page accounting, and properties of the plain restatement that the GPU tests lean
on (block edges, the distance penalty, cut invariance of the recurrence, routing inside kept
groups, the hashed embedding's first-token row)."""
import pytest
import torch

from oracle import tafisun_ref as R


def _cfg():
    att = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 16, "mask": {"size": 20}, "scale": 0.3}
    moe = {"kind": "moe", "expert": {"ff": 40, "limit": 1.0}, "shared": {"ff": 24, "limit": 0.7},
           "router": {"experts": 6, "identity": 3, "top": 3, "scale": 2.0, "groups": {"count": 3, "keep": 2}}}
    return {"architecture": "Tafisun", "width": 96, "vocab": 160, "norm": {"eps": 1e-5},
            "embedding": {"bigram": {"buckets": 61, "mul_prev": 31, "mul_cur": 5}},
            "layers": [{"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": 80}},
                       {"type": "mingru", "mixer": {"width": 72}, "mlp": moe},
                       {"type": "attention", "mixer": dict(att, heads=2, kv_heads=1, mask=None), "mlp": None}]}


def test_config_reader():
    from mi355_decode.config import ModelConfig
    cfg = ModelConfig.from_dict(_cfg())
    spec = cfg.hybrid
    assert cfg.family == "hybrid" and cfg.architecture == "Tafisun" and cfg.vocab_size == 160 and cfg.hidden_size == 96
    assert spec.arrangement == "pre" and spec.norm_vector and spec.sinusoid_base == 10000.0
    assert (spec.bigram.buckets, spec.bigram.mul_prev, spec.bigram.mul_cur) == (61, 31, 5)
    assert [L.kind for L in spec.layers] == ["attention", "mingru", "attention"]
    a, b = spec.layers[0].battn, spec.layers[2].battn
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.block, a.scale, b.block, b.heads) == (6, 2, 16, 16, 20, 0.3, 0, 2)
    assert spec.layers[0].ff == 80 and spec.layers[0].ff_act == "relu2" and spec.layers[2].ff is None
    m = spec.layers[1].moe
    assert (m.experts, m.identity, m.outputs, m.top, m.groups, m.keep, m.ff) == (6, 3, 9, 3, 3, 2, 40)
    assert (m.score, m.group_score, m.weight_scale, m.limit, m.shared_ff, m.shared_limit) == ("softmax", "max", 2.0, 1.0, 24, 0.7)
    assert spec.layers[1].gru.width == 72 and spec.runs() == [(0, None), (1, None), (2, None)]
    for change, where in (({"kv_heads": 4}, 0), ({"vdim": 24}, 0)):    # heads not a multiple; values that cannot be the keys
        bad = _cfg()
        bad["layers"][where]["mixer"].update(change)
        with pytest.raises(ValueError):
            ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][1]["mlp"]["router"]["top"] = 7              # two kept groups of three outputs hold six
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][1]["mlp"]["router"]["identity"] = 2         # eight outputs do not split into three groups
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][1]["type"] = "delta"
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
    assert list(l0.seg) == ["q", "k", "g"] and list(l1.seg) == ["z", "x", "g"]
    for lw in w.layers:
        assert all(a % 8 == 0 for a, _ in lw.seg.values())
    a, n = l0.seg["k"]
    assert n == 32 and torch.equal(l0.in_w[a:a + n], st["l0.mix.k"])
    assert l0.q_norm.dtype == torch.float32 and l0.r1.shape == (6,) and l1.z_b.shape == (72,)
    assert torch.equal(l0.up_w, st["l0.mlp.up"]) and l0.down_w.shape == (96, 80) and l0.gate_up_w is None
    # the shared expert's gate is the last row of the fp32 router matrix
    assert l1.router_w.dtype == torch.float32 and l1.router_w.shape == (10, 96)
    assert torch.equal(l1.router_w[9], st["l1.mlp.shared.sg"][0]) and l1.correction.shape == (9,)
    assert l1.gate_up_w.shape == (6, 80, 96) and torch.equal(l1.gate_up_w[4, 40:], st["l1.mlp.e4.up"])
    assert l1.shared_gate_up_w.shape == (48, 96) and l1.shared_down_w.shape == (96, 24)
    assert l2.norm2 is None and w.bigram.shape == (62, 96)
    # synthetic weights come under the same names
    assert set(W.hybrid_synthetic_state(cfg, seed=0)) == set(st)
    # pages: K and V of the two attention layers, nothing for the recurrence
    runs = [cfg.hybrid.layers[i] for i, _ in cfg.hybrid.runs()]
    assert sum(a.kv_heads * (a.dim + a.vdim) for L in runs for a in (L.attn, L.battn) if a is not None) == 2 * 32 + 1 * 32


def test_restatement_block_edges_penalty_and_first_token_row():
    m = R.block_mask(50, 20)
    for i in range(50):
        assert [j for j in range(50) if m[i, j]] == list(range(i // 20 * 20, i + 1))
    b = R.distance_bias(torch.tensor([0.0, 2.0]), torch.tensor([5.0, 1.0]), 6)
    assert float(b[0].abs().max()) == 0.0 and torch.allclose(b[1, 5, 2], torch.log(torch.tensor(4.0)) * 2)
    # equal scores: the weights fall with the distance as (1 + r2 distance)^(-r1)
    T, d = 8, 4
    q, k = torch.zeros(T, 1, d), torch.zeros(T, 1, d)
    k[:, 0, 0] = torch.arange(T, dtype=torch.float32)
    o = R.block_attention(q, k, torch.ones(d), torch.ones(d), torch.tensor([1.0]), torch.tensor([1.0]), 1.0, 0, 1e-5)
    w = 1.0 / (1.0 + torch.arange(T - 1, -1, -1, dtype=torch.float32))
    assert torch.allclose(o[-1, 0], (w * torch.arange(T)).sum() / w.sum(), atol=1e-5)
    # the hashed embedding: row `buckets` for the first token, the hash of the pair after it
    cfg = {"width": 4, "embedding": {"bigram": {"buckets": 5, "mul_prev": 3, "mul_cur": 2}}}
    wt = {"embed": torch.zeros(9, 4), "bigram": torch.arange(6, dtype=torch.float32)[:, None].expand(6, 4).contiguous()}
    x = R.embed_tokens(wt, cfg, [7, 8, 1])
    pe0 = torch.tensor([0.0, 1.0, 0.0, 1.0])
    assert torch.allclose(x[0], 5.0 + pe0) and torch.allclose(x[1, 0] - torch.sin(torch.tensor(1.0)), torch.tensor(float((7 * 3 + 8 * 2) % 5)))


def test_restatement_recurrence_is_cut_invariant_and_routes_inside_kept_groups():
    g = torch.Generator().manual_seed(0)
    z, c = torch.rand(11, 5, generator=g), R.mingru_candidate(torch.randn(11, 5, generator=g) * 3)
    whole = R.mingru_scan(z, c)
    part = R.mingru_scan(z[4:], c[4:], whole[3])
    assert torch.allclose(part, whole[4:], atol=1e-6)
    u = torch.tensor([-2.0, 0.0, 3.0])
    assert torch.allclose(R.mingru_candidate(u), torch.tensor([float(torch.sigmoid(u[0])), 0.5, 3.5]))
    zl = torch.randn(200, 12, generator=g)
    corr = torch.randn(12, generator=g) * 0.05 - 2.0          # every choice score below zero
    ids, wts = R.route(zl, corr, 3, 4, 2, 1.5)
    s = torch.softmax(zl, dim=-1)
    choice = s + corr
    gs = choice.view(200, 4, 3).max(dim=-1).values
    for t in range(200):
        kept = set(gs[t].topk(2).indices.tolist())
        allowed = [e for e in range(12) if e // 3 in kept]
        assert sorted(ids[t].tolist()) == sorted(sorted(allowed, key=lambda e: -float(choice[t, e]))[:3])
        assert torch.allclose(wts[t], s[t, ids[t]] * 1.5)
