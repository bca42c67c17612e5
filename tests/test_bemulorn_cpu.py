"""The Bemulorn design of the hybrid family without a GPU: the reader of config.json and its
refusals, the weight layout (one input matrix with its bias row, one output matrix over the heads
and the hidden units side by side), page accounting for layers that share pages, the blended
rotary frequencies, and properties of the plain restatement that the GPU tests lean on (chunk
edges, the value-less softmax term, the softmax over the chosen logits, the limited unit)."""
import math

import pytest
import torch

from oracle import bemulorn_ref as R


def _cfg():
    rot = {"dims": 8, "base": 500.0, "scaling": {"factor": 3.0, "original": 40, "fast": 8.0, "slow": 1.5}}
    att = {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "mask": {"size": 20}, "scale": 0.3, "rot": rot}
    moe = {"kind": "moe", "expert": {"ff": 40}, "shared": {"ff": 24}, "router": {"experts": 6, "top": 2}}
    return {"architecture": "Bemulorn", "width": 96, "vocab": 160, "max_positions": 200, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.7}, "logit_scale": 0.6,
            "layers": [{"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": 80, "limit": 1.2}},
                       {"type": "attention", "mixer": dict(att, heads=4, kv_from=0, mask={"size": 7}), "mlp": moe},
                       {"type": "attention", "mixer": dict(att, heads=3, kv_heads=3, vdim=7, mask=None, rot={"dims": 16, "base": 100.0}),
                        "mlp": None}]}


def test_config_reader():
    from mi355_decode.config import ModelConfig
    cfg = ModelConfig.from_dict(_cfg())
    spec = cfg.hybrid
    assert cfg.family == "hybrid" and cfg.architecture == "Bemulorn" and cfg.vocab_size == 160 and cfg.hidden_size == 96
    assert cfg.max_position_embeddings == 200 and cfg.rms_norm_eps == 1e-5
    assert spec.arrangement == "parallel" and spec.norm_vector and spec.learned_positions
    assert (spec.embed_scale, spec.logit_scale) == (1.7, 0.6)
    a, b, c = (L.battn for L in spec.layers)
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.block, a.scale, a.kv_from) == (6, 2, 16, 24, 20, 0.3, None)
    assert (b.heads, b.block, b.kv_from, c.block, c.kv_heads, c.vdim, c.rot_dims, c.rot_base) == (4, 7, 0, 0, 3, 7, 16, 100.0)
    assert not a.values_are_keys and not a.qk_norm and not a.penalty and a.bias and a.sink == 0.0 and a.gate_per_head
    assert (a.rot_dims, a.rot_base) == (8, 500.0) and c.rot_scaling is None
    assert (a.rot_scaling.factor, a.rot_scaling.original, a.rot_scaling.fast, a.rot_scaling.slow) == (3.0, 40.0, 8.0, 1.5)
    assert spec.layers[0].ff == 80 and spec.layers[0].ff_act == "limited" and spec.layers[0].ff_limit == 1.2
    m = spec.layers[1].moe
    assert (m.experts, m.top, m.ff, m.score, m.router_bias, m.shared_ff, m.shared_gated, m.limit) == \
        (6, 2, 40, "chosen_softmax", True, 24, False, None)
    assert spec.layers[2].ff is None and spec.layers[2].moe is None and spec.runs() == [(0, None), (1, None), (2, None)]
    for where, change in ((0, {"kv_heads": 4}), (0, {"rot": {"dims": 18, "base": 10.0}}), (0, {"rot": {"dims": 7, "base": 10.0}}),
                          (1, {"kv_from": 1}), (1, {"kv_from": 2}), (1, {"kv_heads": 1}), (2, {"kv_from": 1})):
        bad = _cfg()
        bad["layers"][where]["mixer"].update(change)
        with pytest.raises(ValueError):
            ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][1]["mlp"]["router"]["top"] = 7
    with pytest.raises(ValueError):
        ModelConfig.from_dict(bad)
    bad = _cfg()
    bad["layers"][1]["type"] = "mingru"
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
    assert list(l0.seg) == ["q", "k", "v", "g", "gate", "up"] and list(l1.seg) == ["q", "g", "gate", "up"]
    assert list(l2.seg) == ["q", "k", "v", "g"]
    for lw in w.layers:
        assert all(a % 8 == 0 for a, _ in lw.seg.values())
    a, n = l0.seg["k"]
    assert n == 32 and torch.equal(l0.in_w[a:a + n], st["l0.mix.k"]) and torch.equal(l0.in_b[a:a + n], st["l0.mix.k.b"])
    a, n = l0.seg["g"]
    assert n == 6 and float(l0.in_b[a:a + 8].abs().max()) == 0.0          # no bias on the gate, zero rows of padding
    a, n = l1.seg["gate"]
    assert n == 24 and torch.equal(l1.in_w[a:a + n], st["l1.mlp.shared.gate"])
    # heads | hidden units side by side; 3 heads of 7 value channels are padded to 24 columns of zeros
    assert l0.out_w.shape == (96, 6 * 24 + 80) and torch.equal(l0.out_w[:, :144], st["l0.mix.o"])
    assert torch.equal(l0.out_w[:, 144:], st["l0.mlp.down"])
    assert l1.out_w.shape == (96, 4 * 24 + 24) and torch.equal(l1.out_w[:, 96:], st["l1.mlp.shared.down"])
    assert l2.out_w.shape == (96, 24) and torch.equal(l2.out_w[:, :21], st["l2.mix.o"]) and float(l2.out_w[:, 21:].abs().max()) == 0.0
    assert l1.router_w.dtype == torch.float32 and l1.router_w.shape == (6, 96) and torch.equal(l1.router_b, st["l1.mlp.router.b"])
    assert float(l1.correction.abs().max()) == 0.0
    assert l1.gate_up_w.shape == (6, 80, 96) and torch.equal(l1.gate_up_w[4, 40:], st["l1.mlp.e4.up"])
    assert l0.sink.shape == (6,) and float(l0.sink.abs().max()) == 0.0 and w.pos_embed.shape == (200, 96)
    # synthetic weights come under the same names
    assert set(W.hybrid_synthetic_state(cfg, seed=0)) == set(st)
    bad = dict(st)
    bad["l1.mix.q.b"] = bad["l1.mix.q.b"][:-1]
    with pytest.raises(ValueError):
        W.from_state_dict(cfg, bad, torch.float32, "cpu")
    # pages: K and V of the two layers that have projections of their own, nothing for the layer that shares
    runs = [cfg.hybrid.layers[i] for i, _ in cfg.hybrid.runs()]
    assert sum(a.kv_heads * (a.dim + a.vdim) for L in runs for a in (L.battn,) if a.kv_from is None) == 2 * 40 + 3 * 23


def test_blended_frequencies():
    from mi355_decode.config import RotaryScaling
    f, mult = RotaryScaling(4.0, 128.0, 32.0, 1.0).frequencies(32, 10000.0)
    plain = [10000.0 ** (-2.0 * i / 32) for i in range(16)]
    c = lambda r: 32 * math.log(128.0 / (2 * math.pi * r)) / (2 * math.log(10000.0))      # noqa: E731
    lo, hi = max(math.floor(c(32.0)), 0), min(math.ceil(c(1.0)), 31)
    assert lo == 0 and 0 < hi < 16                              # (negative before the clamp; the ramp ends inside the pairs)
    for i in range(16):
        m = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        assert abs(f[i] - (plain[i] / 4.0 * m + plain[i] * (1 - m))) < 1e-15
    assert f[0] == 1.0 and abs(f[15] - plain[15] / 4.0) < 1e-18 and abs(mult - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    cos, sin = R.rotary_angles({"dims": 32, "base": 10000.0, "scaling": {"factor": 4.0, "original": 128, "fast": 32.0, "slow": 1.0}},
                               5, torch.float64)
    assert torch.allclose(cos[3], torch.cos(3.0 * torch.tensor(f).float().double()) * mult, atol=1e-12)
    # a factor of one changes nothing
    f1, m1 = RotaryScaling(1.0, 64.0, 16.0, 2.0).frequencies(8, 100.0)
    assert m1 == 1.0 and all(abs(a - 100.0 ** (-2.0 * i / 8)) < 1e-15 for i, a in enumerate(f1))


def test_restatement_chunk_edges_and_the_value_less_term():
    m = R.chunk_mask(50, 20)
    for i in range(50):
        assert [j for j in range(50) if m[i, j]] == list(range(i // 20 * 20, i + 1))
    assert bool(R.chunk_mask(9, 0)[8, 0]) and not bool(R.chunk_mask(9, 0)[0, 8])
    # equal scores of zero: n keys and the extra term share the weight
    T, d, dv = 6, 4, 3
    v = torch.arange(T * dv, dtype=torch.float32).view(T, 1, dv)
    o = R.attend(torch.zeros(T, 2, d), torch.zeros(T, 1, d), v, 1.0, 0)
    assert torch.allclose(o[-1, :dv], v[:, 0].sum(0) / (T + 1)) and torch.allclose(o[-1, dv:], o[-1, :dv])
    assert torch.allclose(R.attend(torch.zeros(T, 2, d), torch.zeros(T, 1, d), v, 1.0, 0, sink=False)[-1, :dv], v[:, 0].mean(0))
    # chunks of 4: position 4 sees itself only, half the weight goes to the extra term
    o = R.attend(torch.zeros(T, 2, d), torch.zeros(T, 1, d), v, 1.0, 4)
    assert torch.allclose(o[4, :dv], v[4, 0] / 2)
    # a closed gate silences its head only
    gate = torch.tensor([[-40.0, 40.0]]).repeat(T, 1)
    o = R.attend(torch.zeros(T, 2, d), torch.zeros(T, 1, d), v, 1.0, 0, gate)
    assert float(o[:, :dv].abs().max()) < 1e-12 and float(o[-1, dv:].abs().max()) > 1.0
    # large scores do not overflow
    q, k = torch.full((2, 1, 1), 30.0), torch.full((2, 1, 1), 30.0)
    assert torch.isfinite(R.attend(q, k, torch.ones(2, 1, 1), 1.0, 0)).all()


def test_restatement_rotation_chosen_softmax_and_limited_unit():
    cos, sin = R.rotary_angles({"dims": 4, "base": 100.0}, 7)
    x = torch.randn(7, 2, 6, generator=torch.Generator().manual_seed(0))
    y = R.rotate(x, cos, sin, 4)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    assert torch.allclose((y[..., :4] ** 2).sum(-1), (x[..., :4] ** 2).sum(-1), atol=1e-5)
    a = 3 * 100.0 ** (-2.0 * 1 / 4)                              # pair (1, 3) at position 3
    assert torch.allclose(y[3, 0, 1], x[3, 0, 1] * math.cos(a) - x[3, 0, 3] * math.sin(a), atol=1e-5)
    assert torch.allclose(y[3, 0, 3], x[3, 0, 3] * math.cos(a) + x[3, 0, 1] * math.sin(a), atol=1e-5)
    z = torch.tensor([[0.0, 3.0, 1.0, 2.0, -5.0]])
    ids, w = R.choose(z, 2)
    assert ids.tolist() == [[1, 3]] and torch.allclose(w, torch.softmax(torch.tensor([[3.0, 2.0]]), -1))
    assert R.choose(z, 1)[1].tolist() == [[1.0]]
    g, u = torch.tensor([-1.0, 0.5, 9.0]), torch.tensor([-9.0, 0.25, 9.0])
    lim = R.limited_unit(g, u, 2.0)
    want = [-1.0 * torch.sigmoid(torch.tensor(-1.702)) * (-2.0 + 1.0), 0.5 * torch.sigmoid(torch.tensor(0.851)) * 1.25,
            2.0 * torch.sigmoid(torch.tensor(3.404)) * 3.0]
    assert torch.allclose(lim, torch.stack(want))
