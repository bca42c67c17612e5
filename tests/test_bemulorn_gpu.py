"""Hybrid decoders of the Bemulorn design on the GPU against the plain float32 restatement in
oracle/bemulorn_ref.py: every mechanism alone -- the scaled embedding with learned positions, the
rotary table with blended frequencies, rotation and page writes (also of queries alone), the
attention inside chunks with the value-less softmax term, per-head gates and unequal key / value
sizes, routing by logits with a softmax over the chosen, the gated activations on column slices,
the mixture with a biased router and an ungated shared expert -- then the whole model through the
engine: whole prompts, token-by-token decoding, portions down to two tokens, mixed batches, reused
pages and slots, chunk and page edges, layers that share pages, other sizes, and greedy generation
through LLM.generate.  Small seeded configurations made here; float32 runs carry the sharp bars,
bfloat16 a loose one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import bemulorn_ref as R  # noqa: E402


def _attn(heads, kv_heads, dim, vdim, size, scale=0.25, rot=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    if rot:
        m["rot"] = rot
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _rot(dims, base=10000.0, factor=None, original=64, fast=16.0, slow=2.0):
    r = {"dims": dims, "base": base}
    if factor:
        r["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return r


def _moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


_RA, _RB = _rot(8, 500.0, 3.0, 40, 8.0, 1.5), _rot(24, 10000.0)
CONFIGS = {
    # heads three to one and one to one, chunks that end inside a page (20, 7), a layer without a
    # feed-forward, two layers that read the pages of layer 0 and one that reads layer 2's, a mixture
    # with and one without a shared expert, values wider and narrower than keys
    "mix": {"architecture": "Bemulorn", "width": 96, "vocab": 160, "max_positions": 320, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.7}, "logit_scale": 0.6,
            "layers": [{"type": "attention", "mixer": _attn(6, 2, 16, 24, 20, 0.3, _RA), "mlp": _dense(80, 1.2)},
                       {"type": "attention", "mixer": _attn(4, 2, 16, 24, 7, 0.2, _RA, kv_from=0), "mlp": _moe(6, 2, 40, shared=24)},
                       {"type": "attention", "mixer": _attn(3, 3, 24, 8, 64, 0.25, _RB), "mlp": None},
                       {"type": "attention", "mixer": _attn(2, 2, 16, 24, 33, 0.3, _RA, kv_from=0), "mlp": _moe(5, 3, 24)},
                       {"type": "attention", "mixer": _attn(6, 3, 24, 8, 0, 0.2, _RB, kv_from=2), "mlp": _dense(56, 0.4)}]},
    # no embedding scale, no logit scale, no rotation in one layer and all of the head in another, a chunk
    # of one position and no chunks at all, one expert chosen and all experts chosen, a head wider than 128
    "plain": {"architecture": "Bemulorn", "width": 64, "vocab": 97, "max_positions": 320, "norm": {"eps": 1e-6},
              "layers": [{"type": "attention", "mixer": _attn(2, 2, 16, 16, 1, 0.3), "mlp": _moe(3, 1, 16)},
                         {"type": "attention", "mixer": _attn(4, 1, 8, 12, 0, 0.4, _rot(8, 100.0)), "mlp": _moe(4, 4, 16, shared=8)},
                         {"type": "attention", "mixer": _attn(1, 1, 136, 40, 40, 0.1, _rot(64, 10000.0, 8.0, 32, 4.0, 1.0)),
                          "mlp": None},
                         {"type": "attention", "mixer": _attn(4, 1, 8, 12, 16, 0.5, _rot(8, 100.0), kv_from=1), "mlp": _dense(24, 7.0)}]},
    # sizes that the matrix-core attention (layers 0 and 1 also its LDS-staged form for prompts: equal key and
    # value sizes of 64), the matrix-core expert rows and (width 512) the tiled weight stream cover in 16 bits
    "wide": {"architecture": "Bemulorn", "width": 512, "vocab": 384, "max_positions": 320, "norm": {"eps": 1e-6},
             "embedding": {"scale": 2.0}, "logit_scale": 1.5,
             "layers": [{"type": "attention", "mixer": _attn(8, 2, 64, 64, 48, 0.125, _rot(32, 10000.0, 4.0, 128, 32.0, 1.0)),
                         "mlp": _moe(8, 2, 256, shared=128)},
                        {"type": "attention", "mixer": _attn(6, 2, 64, 64, 33, 0.1, _rot(32, 10000.0, 4.0, 128, 32.0, 1.0), kv_from=0),
                         "mlp": _dense(1024, 1.5)},
                        {"type": "attention", "mixer": _attn(6, 2, 32, 48, 0, 0.2, _rot(16, 1000.0)), "mlp": _moe(16, 4, 128)}]},
    # a width that is no multiple of 8, head and expert sizes that no matrix-core tile covers, five
    # ungrouped heads, heads * vdim that is no multiple of 8, seven experts of which three run
    "odd": {"architecture": "Bemulorn", "width": 90, "vocab": 101, "max_positions": 320, "norm": {"eps": 1e-5},
            "embedding": {"scale": 0.5}, "logit_scale": 3.0,
            "layers": [{"type": "attention", "mixer": _attn(5, 5, 24, 7, 96, 0.2, _rot(10, 77.0, 2.0, 50, 10.0, 3.0)),
                        "mlp": _moe(5, 2, 30, shared=22)},
                       {"type": "attention", "mixer": _attn(3, 1, 20, 9, 10, 0.3, _rot(20, 10000.0)), "mlp": _dense(50, 2.0)},
                       {"type": "attention", "mixer": _attn(5, 5, 24, 7, 13, 0.2, _rot(10, 77.0, 2.0, 50, 10.0, 3.0), kv_from=0),
                        "mlp": _moe(7, 3, 18)}]},
}
_cache = {}


def _weights(name):
    if ("w", name) not in _cache:
        _cache[("w", name)] = R.random_state(CONFIGS[name], seed=len(name))
    return _cache[("w", name)]


def _engine(name, dtype="float32", pages=40, max_model_len=320):
    from mi355_decode.config import EngineArgs, ModelConfig
    from mi355_decode.llm import build_engine
    key = (name, dtype, pages, max_model_len)
    if key not in _cache:
        torch.backends.cuda.matmul.allow_tf32 = False
        _cache[key] = build_engine(EngineArgs(model=name, dtype=dtype, max_num_seqs=4, max_model_len=max_model_len,
                                              num_gpu_blocks_override=pages, gpu_memory_utilization=0.0,
                                              max_num_batched_tokens=1 << 20),
                                   state_dict=_weights(name), model_config=ModelConfig.from_dict(CONFIGS[name]))
    eng = _cache[key]
    assert not eng.seqs and eng.alloc.num_free == pages and eng.slots.num_free == 4
    return eng


def _tokens(name, n, seed):
    return np.random.default_rng(seed).integers(0, CONFIGS[name]["vocab"], n).tolist()


def _ref(name, toks):
    key = ("ref", name, tuple(toks))
    if key not in _cache:
        with torch.no_grad():
            _cache[key] = R.forward(_weights(name), CONFIGS[name], toks).numpy()
    return _cache[key]


def _close(got, want, tol=3e-4):
    scale = float(np.abs(want).max())
    err = float(np.abs(got - want).max())
    assert err <= tol * scale, f"max |diff| {err:.3e} on a scale of {scale:.3f}"


def _run_cuts(eng, rid, toks, cuts):
    """Feeds toks in portions `cuts` (the last portion takes the rest), all positions wanted."""
    rows, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = min(sizes.pop(0) if sizes else len(toks) - at, len(toks) - at)
        rows.append(eng.forced_step([(rid, toks[at:at + n], list(range(n)))], [rid] if at + n == len(toks) else []))
        at += n
    return np.concatenate(rows)


# ------------------------------------------------------------------------------------------ #
# mechanisms alone
# ------------------------------------------------------------------------------------------ #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,scale", [(10, 1.0), (33, 2.5), (64, 0.125)])
def test_scaled_embedding_with_learned_positions(dtype, W, scale):
    """Packed rows of several sequences at scattered positions: the embedding row is scaled, the
    position row is not."""
    from mi355_decode import ops
    g = torch.Generator().manual_seed(W)
    V, P = 50, 40
    embed, pos = torch.randn(V, W, generator=g).to(dtype), torch.randn(P, W, generator=g).to(dtype)
    ids = torch.randint(0, V, (23,), generator=g)
    positions = torch.tensor([0, 1, 2, 3, 17, 18, 39, 0, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 31, 32, 33])
    got = ops.embed_scale_pos_f32(embed.cuda(), ids.cuda(), scale, pos.cuda(), positions.cuda()).cpu()
    want = embed.float()[ids] * scale + pos.float()[positions]
    assert got.dtype == torch.float32 and (got - want).abs().max() <= 1e-6 * want.abs().max()     # (a fused multiply-add)


@pytest.mark.parametrize("rot", [_rot(8, 500.0), _rot(8, 500.0, 3.0, 40, 8.0, 1.5), _rot(32, 10000.0, 4.0, 128, 32.0, 1.0),
                                 _rot(64, 10000.0, 8.0, 32, 4.0, 1.0), _rot(10, 77.0, 2.0, 50, 10.0, 3.0),
                                 _rot(16, 10000.0, 1.0, 4096, 32.0, 1.0), _rot(6, 20.0, 16.0, 4, 2.0, 1.0)])
def test_rotary_table_with_blended_frequencies(rot):
    """cos | sin rows of the engine's table against the restatement: plain frequencies, blends whose ramp
    covers a part, all or none of the pairs, a factor of one, and a ramp of zero width."""
    from mi355_decode.config import RotaryScaling
    from mi355_decode.hybrid_runner import rotary_table
    sc = rot.get("scaling")
    scaling = RotaryScaling(sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None
    T = 700
    table = rotary_table(rot["dims"], rot["base"], T, "cuda", scaling).cpu()
    cos, sin = R.rotary_angles(rot, T, torch.float64)
    assert table.shape == (T, rot["dims"])
    # float32 angles of several hundred radians carry an absolute error near 3e-5
    assert (table[:, : rot["dims"] // 2] - cos.float()).abs().max() < 2e-4
    assert (table[:, rot["dims"] // 2:] - sin.float()).abs().max() < 2e-4
    assert (table[:20, : rot["dims"] // 2] - cos.float()[:20]).abs().max() < 3e-6


def _pages(T, G, d, dv, dtype, spare=3, seed=0):
    """A shuffled page table for one sequence of T tokens over NaN-filled pools."""
    n = -(-T // 16)
    order = torch.randperm(n + spare, generator=torch.Generator().manual_seed(seed))[:n]
    kc = torch.full((n + spare, G, 16, d), float("nan"), dtype=dtype, device="cuda")
    vc = torch.full((n + spare, G, dv, 16), float("nan"), dtype=dtype, device="cuda")
    bt = order.to(torch.int32).view(1, n).cuda()
    slots = (order[torch.arange(T) // 16] * 16 + torch.arange(T) % 16).cuda()
    return kc, vc, bt, slots


def _attend_in_cuts(q, k, v, gate, cuts, size, scale, rot=None, tiled=False, splits=0, sink=True, staged=False):
    """q [T, H, d], k [T, G, d], v [T, G, dv] unrotated, gate [T, H]: rotation + page write + attention
    through the product's kernels, portion by portion, over shuffled NaN-filled pages; the output lands in
    a column slice of a wider NaN-filled row."""
    from mi355_decode import ops
    from mi355_decode.config import RotaryScaling
    from mi355_decode.hybrid_runner import rotary_table
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    dt = q.dtype
    kc, vc, bt, slots = _pages(T, G, d, dv, dt)
    sc = (rot or {}).get("scaling")
    table = rotary_table(rot["dims"] if rot else 0, rot["base"] if rot else 1.0, T + 16, "cuda",
                         RotaryScaling(sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None)
    sink_t = torch.zeros(H, dtype=torch.float32, device="cuda") if sink else None
    outs, at = [], 0
    cuts = list(cuts) + ([T - sum(cuts)] if sum(cuts) < T else [])        # the last portion takes the rest
    for n in cuts:
        pos = torch.arange(at, at + n, dtype=torch.int64, device="cuda")
        # one buffer as a projection would leave it: q | k | v | gate side by side
        width = (H + G) * d + G * dv + H
        buf = torch.cat([q[at:at + n].reshape(n, -1), k[at:at + n].reshape(n, -1), v[at:at + n].reshape(n, -1),
                         gate[at:at + n], torch.zeros(n, -width % 8, dtype=dt)], dim=1).cuda().contiguous()
        qs, ks = buf[:, : H * d], buf[:, H * d: (H + G) * d]
        vs, gs = buf[:, (H + G) * d: (H + G) * d + G * dv], buf[:, (H + G) * d + G * dv: width]
        ops.rope_partial_kv_write(qs, ks, vs, table, pos, slots[at:at + n], kc, vc, H, G, d, dv)
        tiles = torch.from_numpy(ops.query_tiles(np.array([0, n]))).cuda() if tiled else None
        lead = 8 if staged else 3                                # (the staged form wants 16-byte aligned rows)
        row = torch.full((n, H * dv + 16), float("nan"), dtype=dt, device="cuda")
        if staged:
            assert ops.chunk_attn_prefill_ok(dt, H, G, d, dv)
            ops.paged_attn_prefill_ext(qs, kc, vc, bt, torch.tensor([0, n], dtype=torch.int32, device="cuda"),
                                       torch.tensor([at + n], dtype=torch.int32, device="cuda"), n, H, G, d, scale, chunk=size,
                                       sink=sink_t, gate=gs, out=row[:, lead: lead + H * dv])
        else:
            ops.softmax_bias_attn(qs, kc, vc, bt, torch.zeros(n, dtype=torch.int32, device="cuda"), pos, None, None, gs, H, scale,
                                  block=size, tiles=tiles, num_splits=splits, sink=sink_t, out=row[:, lead: lead + H * dv])
        assert torch.isnan(row[:, :lead]).all() and torch.isnan(row[:, lead + H * dv:]).all()
        outs.append(row[:, lead: lead + H * dv].float().cpu())
        at += n
    return torch.cat(outs)


def _attend_ref(q, k, v, gate, size, scale, rot=None, sink=True):
    T = q.shape[0]
    if rot:
        cos, sin = R.rotary_angles(rot, T)
        q, k = R.rotate(q, cos, sin, rot["dims"]), R.rotate(k, cos, sin, rot["dims"])
    return R.attend(q, k, v, scale, size, gate, sink=sink)


@pytest.mark.parametrize("H,G,d,dv,size,rot", [(6, 2, 16, 24, 20, _RA), (3, 3, 24, 8, 7, _RB), (2, 1, 32, 48, 64, _rot(32, 100.0)),
                                               (4, 4, 20, 20, 1, None), (4, 1, 8, 12, 0, _rot(8, 100.0)),
                                               (1, 1, 136, 40, 40, _rot(64, 10000.0, 8.0, 32, 4.0, 1.0)),
                                               (8, 2, 64, 32, 1000, _rot(32, 10000.0, 4.0, 128, 32.0, 1.0)), (5, 5, 24, 7, 13, None)])
def test_attention_whole_portions_and_single_tokens(H, G, d, dv, size, rot):
    g = torch.Generator().manual_seed(H * 100 + d)
    T = 75
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g)
    gate = torch.randn(T, H, generator=g) * 2
    ref = _attend_ref(q, k, v, gate, size, 0.3, rot)
    for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
        got = _attend_in_cuts(q, k, v, gate, cuts, size, 0.3, rot)
        assert (got - ref).abs().max() <= 3e-5 * ref.abs().max(), cuts
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    got = _attend_in_cuts(b16(q), b16(k), b16(v), b16(gate), [40, 2, 1, 32], size, 0.3, rot)
    ref = _attend_ref(b16(q).float(), b16(k).float(), b16(v).float(), b16(gate).float(), size, 0.3, rot)
    assert (got - ref).abs().max() <= 3e-2 * ref.abs().max()


@pytest.mark.parametrize("H,G,d,dv,size,rot", [(6, 2, 32, 16, 20, _rot(8, 500.0, 3.0, 40, 8.0, 1.5)), (3, 3, 64, 48, 7, _RB),
                                               (8, 2, 64, 32, 48, _rot(32, 10000.0, 4.0, 128, 32.0, 1.0)), (4, 4, 96, 16, 1, None),
                                               (8, 1, 32, 64, 0, _rot(32, 100.0)), (2, 1, 128, 128, 40, _rot(64, 10000.0)),
                                               (5, 1, 64, 48, 33, _rot(32, 10000.0)), (12, 2, 32, 80, 17, None)])
def test_attention_on_the_matrix_cores(H, G, d, dv, size, rot):
    """bfloat16 inputs; the restatement sees the same rounded inputs, so what is left is the rounding of
    the rotated queries and keys in their 16-bit storage and of the weights in the second product.
    Single rows spread their keys over three workgroups, which a second launch joins (the value-less
    term enters there)."""
    g = torch.Generator().manual_seed(H * 100 + d)
    T = 75
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    q, k, v = b16(torch.randn(T, H, d, generator=g)), b16(torch.randn(T, G, d, generator=g)), b16(torch.randn(T, G, dv, generator=g))
    gate = b16(torch.randn(T, H, generator=g) * 2)
    for sink in (True, False):
        ref = _attend_ref(q.float(), k.float(), v.float(), gate.float(), size, 0.3, rot, sink=sink)
        for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
            got = _attend_in_cuts(q, k, v, gate, cuts, size, 0.3, rot, tiled=True, splits=3, sink=sink)
            assert (got - ref).abs().max() <= 3e-2 * ref.abs().max(), (cuts, sink)


@pytest.mark.parametrize("T", [75, 300])
@pytest.mark.parametrize("H,G,d,size,rot", [(8, 2, 64, 48, _rot(32, 10000.0, 4.0, 128, 32.0, 1.0)), (4, 4, 64, 7, _RB), (16, 4, 128, 20, _RA),
                                            (6, 1, 128, 0, _rot(64, 10000.0)), (3, 1, 64, 33, None), (16, 1, 64, 100, _rot(64, 100.0)),
                                            (2, 2, 128, 1, None), (12, 3, 128, 64, _rot(32, 500000.0)), (5, 1, 64, 128, _RA)])
def test_attention_staged_through_lds(H, G, d, size, rot, T):
    """The form for prompts and portions (equal key and value sizes of 64 or 128, bfloat16): K/V steps staged
    through LDS for a workgroup's tile of queries.  Chunks that end inside a step, a tile and a page; walks
    that start several steps into the sequence; portions that begin and end anywhere; with and without the
    value-less term."""
    g = torch.Generator().manual_seed(H * 100 + d + T)
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    q, k, v = b16(torch.randn(T, H, d, generator=g)), b16(torch.randn(T, G, d, generator=g)), b16(torch.randn(T, G, d, generator=g))
    gate = b16(torch.randn(T, H, generator=g) * 2)
    for sink in (True, False):
        ref = _attend_ref(q.float(), k.float(), v.float(), gate.float(), size, 0.3, rot, sink=sink)
        for cuts in ([T], [2, 3, 1, 30, 2, 16, 21], [T // 2 + 3, 1, 1, 2]) + (([1] * T,) if T == 75 and sink else ()):
            got = _attend_in_cuts(q, k, v, gate, cuts, size, 0.3, rot, staged=True, sink=sink)
            assert (got - ref).abs().max() <= 3e-2 * ref.abs().max(), (cuts, sink)


@pytest.mark.parametrize("size", [16, 17, 31, 48, 64, 65, 400])
def test_chunk_edge_shows_with_one_loud_key(size):
    """The first token of the second chunk holds a key that every query scores far above all others
    and above the value-less term, and a value unlike any other: queries see it exactly while they are
    in that chunk (for the widest chunk: one key among four hundred, two dozen pages back), and the
    last token of the first chunk never does."""
    H, G, d, dv = 2, 1, 32, 16
    j0, T = size, 2 * size + 6
    g = torch.Generator().manual_seed(size)
    q, k, v = torch.zeros(T, H, d), torch.randn(T, G, d, generator=g) * 0.1, torch.randn(T, G, dv, generator=g) * 0.1
    k[:, :, 30] = 0.0                                        # (an unrotated coordinate: rotation covers the first 8)
    k[j0, 0] = 0.0
    k[j0, 0, 30] = 4.0
    q[:, :, 30] = 4.0                                        # score 16 on that key, near 0 on all others
    v[:, :, 5] = 0.0
    v[j0, 0, 5] = 5.0
    gate = torch.full((T, H), 20.0)                          # an open gate
    rot = _rot(8, 100.0, 2.0, 16, 4.0, 1.0)
    ref = _attend_ref(q, k, v, gate, size, 1.0, rot)
    last_in, first_out = 2 * size - 1, 2 * size
    assert float(ref[last_in, 5]) > 4.9 and float(ref[last_in, dv + 5]) > 4.9          # both heads, the far end of the chunk
    assert abs(float(ref[first_out, 5])) < 1e-3 and abs(float(ref[j0 - 1, 5])) < 1e-3  # the next chunk; the chunk before
    for cuts in ([T], [last_in, 1, 1] + [1] * 5, [5, 2] + [1] * (T - 7), [j0, 1, 2, 2]):
        got = _attend_in_cuts(q, k, v, gate, cuts, size, 1.0, rot)
        assert (got - ref).abs().max() <= 1e-4 * ref.abs().max(), cuts
        b16 = lambda t: t.to(torch.bfloat16)                  # noqa: E731
        got = _attend_in_cuts(b16(q), b16(k), b16(v), b16(gate), cuts, size, 1.0, rot, tiled=True, splits=4)
        r16 = _attend_ref(b16(q).float(), b16(k).float(), b16(v).float(), b16(gate).float(), size, 1.0, rot)
        assert (got - r16).abs().max() <= 3e-2 * r16.abs().max(), cuts
    # the same key through the LDS-staged form (equal key and value sizes of 64): pad both with silent channels
    q6, k6, v6 = torch.zeros(T, H, 64), torch.zeros(T, G, 64), torch.zeros(T, G, 64)
    q6[..., :d], k6[..., :d], v6[..., :dv] = q, k, v
    r16 = _attend_ref(b16(q6).float(), b16(k6).float(), b16(v6).float(), b16(gate).float(), size, 1.0, rot)
    assert float(r16[last_in, 5]) > 4.9 and abs(float(r16[first_out, 5])) < 1e-3
    for cuts in ([T], [last_in, 1, 1], [5, 2, j0 - 7, 1, 2, 2], [j0 + 1, size - 2, 1, 1]):
        got = _attend_in_cuts(b16(q6), b16(k6), b16(v6), b16(gate), cuts, size, 1.0, rot, staged=True)
        assert (got - r16).abs().max() <= 3e-2 * r16.abs().max(), cuts


def test_value_less_term_takes_its_share_of_the_weight():
    """All scores zero: n visible keys and the extra term share the weight equally, so the output is
    the sum of the values over n + 1 (a plain softmax would give their mean).  All scores far below
    zero: the extra term takes everything and the output vanishes."""
    H, G, d, dv, T = 2, 1, 32, 16, 40
    g = torch.Generator().manual_seed(1)
    v = torch.randn(T, G, dv, generator=g)
    q, k, gate = torch.zeros(T, H, d), torch.zeros(T, G, d), torch.full((T, H), 30.0)
    n = torch.arange(1, T + 1, dtype=torch.float32)[:, None]
    want = (torch.cumsum(v[:, 0], dim=0) / (n + 1)).repeat(1, H)
    for kw in (dict(), dict(tiled=True, splits=2)):
        dt = torch.bfloat16 if kw else torch.float32
        got = _attend_in_cuts(q.to(dt), k.to(dt), v.to(dt), gate.to(dt), [T], 0, 1.0, **kw)
        assert (got - want).abs().max() <= (2e-2 if kw else 1e-5)
        plain = _attend_in_cuts(q.to(dt), k.to(dt), v.to(dt), gate.to(dt), [T], 0, 1.0, sink=False, **kw)
        assert (plain - want * (n + 1) / n).abs().max() <= (2e-2 if kw else 1e-5)
        q2, k2 = q.clone(), k.clone()
        q2[:, :, 0], k2[:, :, 0] = 6.0, -6.0                   # every score -36
        got = _attend_in_cuts(q2.to(dt), k2.to(dt), v.to(dt), gate.to(dt), [10, 1, 29], 0, 1.0, **kw)
        assert got.abs().max() < 1e-10


def test_queries_alone_rotate_and_leave_the_pages():
    """A layer that reads another layer's pages rotates its queries and writes nothing."""
    from mi355_decode import ops
    from mi355_decode.hybrid_runner import rotary_table
    H, G, d, dv, T = 3, 1, 16, 8, 21
    g = torch.Generator().manual_seed(3)
    q = torch.randn(T, H * d + 5, generator=g)
    table = rotary_table(8, 50.0, 64, "cuda")
    pos = torch.arange(30, 30 + T, dtype=torch.int64)
    qd = q.cuda()
    ops.rope_partial_kv_write(qd[:, : H * d], None, None, table, pos.cuda(), torch.zeros(T, dtype=torch.int64, device="cuda"),
                              None, None, H, G, d, dv)
    cos, sin = R.rotary_angles(_rot(8, 50.0), 64)
    want = R.rotate(q[:, : H * d].view(T, H, d), cos[pos], sin[pos], 8).reshape(T, H * d)
    assert (qd[:, : H * d].cpu() - want).abs().max() < 1e-5
    assert torch.equal(qd[:, H * d:].cpu(), q[:, H * d:])


@pytest.mark.parametrize("E,top", [(3, 1), (4, 4), (8, 3), (7, 3), (64, 6), (130, 5), (600, 2)])
def test_routing_by_logits_with_a_softmax_over_the_chosen(E, top):
    from mi355_decode import ops
    g = torch.Generator().manual_seed(E)
    z = torch.randn(37, E + 2, generator=g) * 3              # rows carry two columns more than router outputs
    z[5, :E] = -80.0 - 0.01 * torch.arange(E)                # far below zero: the weights still sum to one
    z[5, 1] = -79.0
    ids, wts = ops.moe_route(z.cuda(), torch.zeros(E, device="cuda"), top, 1, 1, experts=E, chosen_softmax=True)
    rid, rw = R.choose(z[:, :E], top)
    assert torch.equal(ids.cpu().long().sort(dim=1).values, rid.sort(dim=1).values)
    order_g, order_r = ids.cpu().long().argsort(dim=1), rid.argsort(dim=1)
    assert (wts.cpu().gather(1, order_g) - rw.gather(1, order_r)).abs().max() < 1e-6
    assert (wts.cpu().sum(1) - 1).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("limit", [None, 0.4, 7.0])
@pytest.mark.parametrize("F", [27, 32])                     # (32: eight hidden units per thread in 16 bits)
def test_gated_activation_on_column_slices(dtype, limit, F):
    from mi355_decode import ops
    g = torch.Generator().manual_seed(5)
    T = 19
    buf = (torch.randn(T, 8 + 2 * 32, generator=g) * 3).to(dtype)
    gate, up = buf[:, 8: 8 + F], buf[:, 40: 40 + F]
    row = torch.full((T, 40), float("nan"), dtype=dtype, device="cuda")
    d = buf.cuda()
    ops.gated_act_rows(d[:, 8: 8 + F], d[:, 40: 40 + F], limit, out=row[:, 8: 8 + F])
    want = R.silu_unit(gate.float(), up.float()) if limit is None else R.limited_unit(gate.float(), up.float(), limit)
    assert torch.isnan(row[:, :8]).all() and torch.isnan(row[:, 8 + F:]).all()
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert (row[:, 8: 8 + F].float().cpu() - want).abs().max() <= tol * want.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 5, 300])
@pytest.mark.parametrize("W,E,top,F,S", [(72, 6, 2, 40, 24), (96, 5, 3, 64, 0), (64, 4, 4, 16, 8), (64, 3, 1, 32, 0)])
def test_mixture_with_a_biased_router_and_an_ungated_shared_expert(dtype, T, W, E, top, F, S):
    """One layer's feed-forward through the runner's mixture object (300 tokens take the library-GEMM
    path, fewer the row kernels); the rows the caller adds stand for the other sub-layer's output."""
    from mi355_decode.config import MoESpec
    from mi355_decode.hybrid_runner import MoEFeedForward
    g = torch.Generator().manual_seed(W + T)
    mlp = _moe(E, top, F, shared=S or None)
    wt = {"router": torch.randn(E, W, generator=g) * 2 * W ** -0.5, "router.b": torch.randn(E, generator=g) * 0.5}
    for e in range(E):
        wt[f"e{e}.gate"], wt[f"e{e}.up"] = torch.randn(F, W, generator=g) * W ** -0.5, torch.randn(F, W, generator=g) * W ** -0.5
        wt[f"e{e}.down"] = torch.randn(W, F, generator=g) * F ** -0.5
    if S:
        wt["shared.gate"], wt["shared.up"] = torch.randn(S, W, generator=g) * W ** -0.5, torch.randn(S, W, generator=g) * W ** -0.5
        wt["shared.down"] = torch.randn(W, S, generator=g) * S ** -0.5
    wt = {k: v.to(dtype).float() for k, v in wt.items()}
    h = torch.randn(T, W, generator=g).to(dtype)
    other = torch.randn(T, W, generator=g).to(dtype)
    want = R.mixture(wt, "", mlp, h.float()) + other.float()

    class LW:
        pass
    lw = LW()
    put = lambda t: t.to(dtype).cuda().contiguous()          # noqa: E731
    lw.router_w, lw.router_b = wt["router"].cuda(), wt["router.b"].cuda()
    lw.correction = torch.zeros(E, device="cuda")
    lw.gate_up_w = put(torch.stack([torch.cat([wt[f"e{e}.gate"], wt[f"e{e}.up"]]) for e in range(E)]))
    lw.down_w = put(torch.stack([wt[f"e{e}.down"] for e in range(E)]))

    class Rn:
        def linear(self, x, w):
            return x @ w.t()
    spec = MoESpec(experts=E, top=top, groups=1, keep=1, ff=F, score="chosen_softmax", router_bias=True, shared_gated=False)
    shared = other.cuda()
    if S:
        a = R.silu_unit(h.float() @ wt["shared.gate"].T, h.float() @ wt["shared.up"].T).to(dtype)
        shared = (other.float() + a.float() @ wt["shared.down"].T).to(dtype).cuda()
    got = MoEFeedForward(spec, lw, Rn())(h.cuda(), shared=shared).float().cpu()
    if dtype == torch.float32:
        assert (got - want).abs().max() <= 2e-5 * want.abs().max()
    else:
        # rounding may turn a close call of the router: a few rows may differ, the rest must be close
        err = (got - want).abs().amax(1) / want.abs().max()
        assert (err > 5e-2).sum() <= max(T // 50, 0) and err.median() < 2e-2


# ------------------------------------------------------------------------------------------ #
# the whole model through the engine
# ------------------------------------------------------------------------------------------ #
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_every_layer(name):
    eng = _engine(name)
    toks = _tokens(name, 90, 1)
    eng.runner.layer_trace = []
    try:
        got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])
        trace = [t.cpu().numpy() for t in eng.runner.layer_trace]
    finally:
        eng.runner.layer_trace = None
    want = []
    with torch.no_grad():
        R.forward(_weights(name), CONFIGS[name], toks, layers_out=want)
    assert len(trace) == len(want)
    for i, (a, b) in enumerate(zip(trace, want)):
        assert np.abs(a - b.numpy()).max() <= 1e-4 * np.abs(b.numpy()).max(), f"layer {i}"
    _close(got, _ref(name, toks))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_portions_and_token_by_token_equal_the_whole_prompt(name):
    eng = _engine(name)
    toks = _tokens(name, 70, 2)
    want = _ref(name, toks)
    for cuts in ([1] * 70, [2, 2, 3, 16, 1, 17, 2], [33, 2] + [1] * 35, [5] * 14):
        _close(_run_cuts(eng, "p", toks, cuts), want)


def test_first_tokens_and_one_token_requests():
    eng = _engine("mix")
    for n in (1, 2, 3):
        toks = _tokens("mix", n, 10 + n)
        _close(_run_cuts(eng, "s", toks, [1] * n), _ref("mix", toks))
        _close(_run_cuts(eng, "s", toks, [n]), _ref("mix", toks))


def _run_mixed(eng, name):
    """Four requests of unequal length advance together, portions beside single tokens; requests end and new
    ones take their pages and slots.  Returns {request: (tokens, logits of all its positions)}."""
    lens = {"a": 60, "b": 23, "c": 91, "d": 2, "e": 47, "f": 35}
    toks = {r: _tokens(name, n, ord(r)) for r, n in lens.items()}
    plan = {"a": [30, 1, 1, 2, 26], "b": [2, 1, 20], "c": [16, 17, 1, 1, 1, 55], "d": [1, 1], "e": [2, 45], "f": [34, 1]}
    at = {r: 0 for r in lens}
    got = {r: [] for r in lens}
    live, waiting = ["a", "b", "c", "d"], ["e", "f"]
    step = 0
    while live:
        entries, end = [], []
        for r in list(live):
            if r == "b" and step % 2 == 1:
                continue                                            # b sits out every other step
            n = plan[r].pop(0)
            entries.append((r, toks[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == lens[r]:
                end.append(r)
        out = eng.forced_step(entries, end)
        row = 0
        for r, t, _ in entries:
            got[r].append(out[row:row + len(t)])
            row += len(t)
        for r in end:
            live.remove(r)
            if waiting:
                live.append(waiting.pop(0))
        step += 1
    return {r: (toks[r], np.concatenate(got[r])) for r in lens}


@pytest.mark.parametrize("name", ["mix", "plain"])
def test_mixed_batches_equal_each_request_alone(name):
    for toks, got in _run_mixed(_engine(name, pages=24), name).values():
        _close(got, _ref(name, toks))


def test_mixed_batches_in_bfloat16_through_the_staged_attention():
    """The same schedule in bfloat16 on the configuration whose first two layers take the LDS-staged
    attention for steps that hold a portion (single tokens of other requests ride along in that launch)
    and the tile form for steps of single tokens only."""
    name = "wide"
    for toks, got in _run_mixed(_engine(name, dtype="bfloat16", pages=24), name).values():
        want = _ref(name, toks)
        d = got - want
        d = d - d.mean(1, keepdims=True)
        err = np.sqrt((d ** 2).mean(1)) / want.std()
        assert np.median(err) < 0.03 and (err > 0.1).sum() <= max(len(toks) // 12, 1), (np.median(err), np.sort(err)[-6:])


def test_pages_are_reused_without_leaking():
    eng = _engine("plain", pages=8, max_model_len=128)              # one 100-token request nearly fills the pool
    for i in range(6):
        toks = _tokens("plain", 100 - 7 * i, 50 + i)
        _close(_run_cuts(eng, f"r{i}", toks, [40, 3] + [1] * 10), _ref("plain", toks))


def test_long_decoding_past_chunks_and_pages():
    eng = _engine("mix")
    toks = _tokens("mix", 300, 9)
    _close(_run_cuts(eng, "long", toks, [10] + [1] * 290), _ref("mix", toks), tol=6e-4)


def test_a_far_key_through_a_layer_that_shares_pages():
    """Whole model, one attention layer and one that reads its pages, no chunks: the value of token 2
    is made loud through the weights (one value channel of layer 0 answers only to one token's
    embedding), and both layers still hear it 250 tokens later, decoded token by token."""
    cfg = {"architecture": "Bemulorn", "width": 32, "vocab": 40, "max_positions": 320, "norm": {"eps": 1e-6},
           "layers": [{"type": "attention", "mixer": _attn(2, 1, 16, 8, 0, 1.0, _rot(4, 100.0)), "mlp": None},
                      {"type": "attention", "mixer": _attn(2, 1, 16, 8, 0, 1.0, _rot(4, 100.0), kv_from=0), "mlp": None}]}
    from mi355_decode.config import EngineArgs, ModelConfig
    from mi355_decode.llm import build_engine
    w = R.random_state(cfg, seed=11)
    loud = 7
    w["embed"][loud] = 0.0
    w["embed"][loud, 3] = 8.0                               # only token `loud` lights coordinate 3 this much
    w["pos"] *= 0.05
    for i in range(2):
        w[f"l{i}.norm1"][:] = 1.0
    w["l0.mix.k"][:] = 0.0
    w["l0.mix.k"][8, 3] = 4.0                               # an unrotated key coordinate follows coordinate 3
    w["l0.mix.k.b"][:] = 0.0
    for i in range(2):
        w[f"l{i}.mix.q"][:] = 0.0
        w[f"l{i}.mix.q.b"][:] = 0.0
        w[f"l{i}.mix.q.b"][8], w[f"l{i}.mix.q.b"][16 + 8] = 1.5, 1.5     # every query asks for that coordinate
    toks = [int(t) for t in np.random.default_rng(4).integers(8, 40, 260)]
    toks[2] = loud
    torch.backends.cuda.matmul.allow_tf32 = False
    eng = build_engine(EngineArgs(model="far", dtype="float32", max_num_seqs=4, max_model_len=320, num_gpu_blocks_override=20,
                                  gpu_memory_utilization=0.0, max_num_batched_tokens=1 << 20), state_dict=w,
                       model_config=ModelConfig.from_dict(cfg))
    with torch.no_grad():
        want = R.forward(w, cfg, toks).numpy()
        quiet = list(toks)
        quiet[2] = 9
        assert np.abs(R.forward(w, cfg, quiet).numpy()[-1] - want[-1]).max() > 0.05 * np.abs(want[-1]).max()
    _close(_run_cuts(eng, "f", toks, [5] + [1] * 255), want)
    _close(_run_cuts(eng, "f", toks, [200, 2, 58]), want)


@pytest.mark.parametrize("name", ["mix", "wide"])
def test_bfloat16_tracks_the_float32_restatement(name):
    """Whole prompts (library GEMMs, the matrix-core attention) and decode-sized steps (at width 512
    the tiled weight stream, the matrix-core expert rows) in bfloat16 against the restatement and
    against each other.  Rounding may turn a close call of a router, which moves that position's
    logits by far more than rounding does: a few such positions are allowed, the rest must be close."""
    eng = _engine(name, dtype="bfloat16")
    if name == "wide":
        assert eng.runner._tiled_w, "no tiled weight copies at width 512"
    toks = _tokens(name, 64, 4)
    want = _ref(name, toks)
    whole = _run_cuts(eng, "h", toks, [64])
    for got in (whole, _run_cuts(eng, "h", toks, [30, 2] + [1] * 32)):
        for a, b in ((got, want), (got, whole)):
            d = a - b
            d = d - d.mean(1, keepdims=True)
            err = np.sqrt((d ** 2).mean(1)) / want.std()
            assert np.median(err) < 0.03 and (err > 0.1).sum() <= 4, (np.median(err), np.sort(err)[-6:])


@pytest.mark.parametrize("name,dtype", [("mix", "float32"), ("plain", "float32"), ("wide", "bfloat16")])
def test_greedy_generation_through_the_engine(name, dtype):
    """LLM.generate: scheduler admission, prefill, then decode steps replayed from HIP graphs with
    run-ahead.  A token may leave the restatement's only where its own margin is inside the error."""
    from mi355_decode.llm import LLM
    from mi355_decode.sampling_params import SamplingParams
    eng = _engine(name, dtype=dtype)
    prompts = [_tokens(name, n, 70 + n) for n in (5, 33, 18, 1, 26)]     # five requests on four slots: one waits
    steps = 24
    outs = LLM(eng).generate(prompts, SamplingParams(max_tokens=steps, temperature=0.0, ignore_eos=True))
    assert eng.runner.use_graphs and eng.runner.graphs, "the decode steps did not run as HIP graphs"
    tol = 2e-3 if dtype == "float32" else 0.3
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        with torch.no_grad():
            z = R.forward(_weights(name), CONFIGS[name], p + o)[len(p) - 1: -1]
        for t in range(steps):
            best = int(torch.argmax(z[t]))
            assert o[t] == best or float(z[t, best] - z[t, o[t]]) <= tol, f"token {t}: {o[t]} vs {best}"


def test_served_from_a_model_directory(tmp_path):
    """The OpenAI server started on a directory with config.json + model.safetensors of this design: the
    model class chosen by config.json, weights from the checkpoint names, greedy completions by token
    id against the restatement (margin rule), and a seeded sampled completion through the sampler."""
    import json
    import os
    import signal
    import socket
    import subprocess
    import sys
    import time
    from safetensors.torch import save_file
    from conftest import PKG, ROOT
    from mi355_decode.harness import BenchClient
    name = "mix"
    cfg, w = CONFIGS[name], _weights(name)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    json.dump(cfg, open(model_dir / "config.json", "w"))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(model_dir / "model.safetensors"))
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    args = ["--model", str(model_dir), "--served-model-name", "chunks", "--host", "127.0.0.1", "--port", str(port),
            "--dtype", "float32", "--max-num-seqs", "4", "--max-model-len", "128"]
    env = dict(os.environ, PYTHONPATH=PKG + os.pathsep + ROOT)
    log = open(tmp_path / "server.log", "w")
    proc = subprocess.Popen([sys.executable, "-m", "mi355_decode.entrypoints.openai.api_server"] + args, env=env, stdout=log,
                            stderr=subprocess.STDOUT, start_new_session=True)
    url = f"http://127.0.0.1:{port}"
    try:
        client = BenchClient(url)
        t0 = time.time()
        while True:
            assert proc.poll() is None, open(tmp_path / "server.log").read()[-3000:]
            try:
                if client.health() == 200:
                    break
            except Exception:
                pass
            assert time.time() - t0 < 240, "server did not become healthy"
            time.sleep(0.2)
        post = lambda **body: client.http.post(f"{url}/v1/completions", json={"model": "chunks", **body})   # noqa: E731
        prompt, steps = _tokens(name, 21, 5), 12
        r = post(prompt=prompt, max_tokens=steps, temperature=0, ignore_eos=True, logprobs=0, return_tokens_as_token_ids=True)
        assert r.status_code == 200, r.text
        got = [int(t.split(":")[1]) for t in r.json()["choices"][0]["logprobs"]["tokens"]]
        assert len(got) == steps
        with torch.no_grad():
            z = R.forward(w, cfg, prompt + got)[len(prompt) - 1: -1]
        for t in range(steps):
            best = int(torch.argmax(z[t]))
            assert got[t] == best or float(z[t, best] - z[t, got[t]]) <= 2e-3, f"token {t}"
        draws = [post(prompt=prompt, max_tokens=8, temperature=0.9, top_k=20, seed=7, ignore_eos=True, logprobs=0,
                      return_tokens_as_token_ids=True).json()["choices"][0]["logprobs"]["tokens"] for _ in range(2)]
        assert draws[0] == draws[1] and len(draws[0]) == 8
        assert "synthetic" not in open(tmp_path / "server.log").read()
    finally:
        os.killpg(proc.pid, signal.SIGTERM)
        try:
            proc.wait(timeout=20)
        except subprocess.TimeoutExpired:
            os.killpg(proc.pid, signal.SIGKILL)


def test_trace_replay_program(tmp_path):
    """bin/trace_run on a model directory of this design: steps as JSON lines on standard input (a
    portion beside a single token, a request that ends and one that takes its place), float32 logits
    of the wanted rows per step on disk, a 'done <step>' line after every step."""
    import json
    import os
    import subprocess
    from safetensors.torch import save_file
    from conftest import ROOT
    name = "plain"
    cfg, w = CONFIGS[name], _weights(name)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    json.dump(cfg, open(model_dir / "config.json", "w"))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, str(model_dir / "model.safetensors"))
    a, b, c = _tokens(name, 50, 1), _tokens(name, 20, 2), _tokens(name, 9, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}, {"id": "b", "tokens": b[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[1:], "want": [18]}, {"id": "a", "tokens": a[33:34], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[34:36], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [8]}, {"id": "a", "tokens": a[36:], "want": [13]}], "end": ["a", "c"]}]
    p = subprocess.Popen([os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                          "--max-tokens", "128"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            while True:
                line = p.stdout.readline()
                assert line, "the program ended early"
                if line.strip() == f"done {st['step']}":
                    break
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()
    V = cfg["vocab"]
    ra, rb, rc = _ref(name, a), _ref(name, b), _ref(name, c)
    want = {0: [ra[0], ra[32], rb[0]], 1: [rb[19], ra[33]], 3: [rc[8], ra[49]]}
    assert not (out_dir / "2.f32").exists()
    for n, rows in want.items():
        got = np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(-1, V)
        assert got.shape[0] == len(rows)
        _close(got, np.stack(rows))
