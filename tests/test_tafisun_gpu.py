"""Hybrid decoders of the Tafisun design on the GPU against the plain float32 restatement in
oracle/tafisun_ref.py: every mechanism alone -- the hashed previous-token embedding with sinusoidal
positions, the block attention with its distance penalty, the per-channel gated recurrence, softmax
routing with identity experts, the limited expert activation and the shared expert -- then the
whole model through the engine: whole prompts, token-by-token decoding, portions down to two tokens,
mixed batches, reused pages and state slots, block and page edges, other sizes, and greedy
generation through LLM.generate.  Small seeded configurations made here; float32 runs carry the
sharp bars, bfloat16 a loose one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import tafisun_ref as R  # noqa: E402


def _attn(heads, kv_heads, dim, size, scale=0.25):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    return m


def _moe(experts, identity, top, count, keep, ff, limit, scale=1.0, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}
    if shared:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def _bigram(buckets, mul_prev, mul_cur):
    return {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}


CONFIGS = {
    # grouped heads three to one and one to one, blocks that end inside a page (20, 7), a layer without a
    # feed-forward, identity experts, two of three groups kept, a shared expert with its own limit
    "mix": {"architecture": "Tafisun", "width": 96, "vocab": 160, "norm": {"eps": 1e-5}, "embedding": _bigram(61, 31, 5),
            "layers": [{"type": "attention", "mixer": _attn(6, 2, 16, 20, 0.3), "mlp": {"kind": "dense", "ff": 80}},
                       {"type": "mingru", "mixer": {"width": 72}, "mlp": _moe(6, 3, 3, 3, 2, 40, 1.0, 2.0, shared=(24, 0.7))},
                       {"type": "attention", "mixer": _attn(3, 3, 24, 7), "mlp": None},
                       {"type": "mingru", "mixer": {"width": 40}, "mlp": {"kind": "dense", "ff": 56}},
                       {"type": "attention", "mixer": _attn(2, 1, 32, 64, 0.2), "mlp": _moe(5, 0, 2, 1, 1, 24, 3.0)}]},
    # recurrences first, one bucket, a block of one position and no block at all, one identity expert,
    # one expert chosen, weights not scaled, a head wider than 128
    "plain": {"architecture": "Tafisun", "width": 64, "vocab": 97, "norm": {"eps": 1e-6}, "embedding": _bigram(1, 1, 1),
              "layers": [{"type": "mingru", "mixer": {"width": 33}, "mlp": _moe(3, 1, 1, 1, 1, 16, 0.5)},
                         {"type": "mingru", "mixer": {"width": 130}, "mlp": None},
                         {"type": "attention", "mixer": _attn(2, 2, 16, 1), "mlp": {"kind": "dense", "ff": 24}},
                         {"type": "attention", "mixer": _attn(4, 1, 8, 0, 0.4), "mlp": _moe(4, 4, 4, 2, 2, 16, 2.5, 0.5, shared=(8, 9.0))},
                         {"type": "attention", "mixer": _attn(1, 1, 136, 40, 0.1), "mlp": None}]},
    # sizes that the matrix-core attention, the matrix-core expert rows and (width 512) the tiled weight
    # stream cover in 16 bits
    "wide": {"architecture": "Tafisun", "width": 512, "vocab": 384, "norm": {"eps": 1e-6}, "embedding": _bigram(1021, 37, 11),
             "layers": [{"type": "attention", "mixer": _attn(8, 2, 64, 48, 0.125), "mlp": _moe(8, 2, 2, 5, 2, 256, 2.0, 1.5, shared=(128, 1.5))},
                        {"type": "mingru", "mixer": {"width": 512}, "mlp": {"kind": "dense", "ff": 1024}},
                        {"type": "attention", "mixer": _attn(6, 2, 32, 33, 0.2), "mlp": _moe(16, 0, 4, 4, 1, 128, 4.0)}]},
    # a width that is no multiple of 8, head and expert sizes that no matrix-core tile covers, five ungrouped heads,
    # an eight-channel recurrence, seven experts of which three run
    "odd": {"architecture": "Tafisun", "width": 90, "vocab": 101, "norm": {"eps": 1e-5}, "embedding": _bigram(97, 11, 3),
            "layers": [{"type": "mingru", "mixer": {"width": 77}, "mlp": _moe(5, 1, 2, 2, 1, 30, 1.5, 1.2, shared=(22, 1.0))},
                       {"type": "attention", "mixer": _attn(5, 5, 24, 96), "mlp": {"kind": "dense", "ff": 50}},
                       {"type": "attention", "mixer": _attn(4, 2, 48, 10), "mlp": _moe(7, 0, 3, 1, 1, 18, 2.0)},
                       {"type": "mingru", "mixer": {"width": 8}, "mlp": None}]},
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


def _cu(lens):
    return torch.from_numpy(np.cumsum([0] + list(lens)).astype(np.int32)).cuda()


def _i32(v):
    return torch.tensor(list(v), dtype=torch.int32, device="cuda")


# ------------------------------------------------------------------------------------------ #
# mechanisms alone
# ------------------------------------------------------------------------------------------ #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,buckets,mp,mc", [(10, 7, 3, 2), (33, 1, 1, 1), (64, 1021, 100003, 7919)])
def test_embedding_with_previous_token_hash_and_positions(dtype, W, buckets, mp, mc):
    """Two sequences packed side by side, in portions: the previous token of a portion's first row
    comes from the sequence's state slot; a sequence that starts again on a used slot takes the
    first-token row."""
    from mi355_decode import ops
    g = torch.Generator().manual_seed(W)
    V = 50
    wt = {"embed": torch.randn(V, W, generator=g).to(dtype).float(), "bigram": torch.randn(buckets + 1, W, generator=g).to(dtype).float()}
    cfg = {"width": W, "embedding": _bigram(buckets, mp, mc)}
    a, b = torch.randint(0, V, (700,), generator=g).tolist(), torch.randint(0, V, (9,), generator=g).tolist()
    ra, rb = R.embed_tokens(wt, cfg, a), R.embed_tokens(wt, cfg, b)
    emb, big = wt["embed"].to(dtype).cuda(), wt["bigram"].to(dtype).cuda()
    freq = torch.from_numpy((10000.0 ** (-2.0 * np.arange((W + 1) // 2) / W)).astype(np.float32)).cuda()
    prev = torch.full((4,), 12345, dtype=torch.int32, device="cuda")     # junk: position 0 must not read it

    def step(chunks):
        """chunks: [(tokens, first position, slot)]"""
        ids = torch.tensor([t for c in chunks for t in c[0]], dtype=torch.int64, device="cuda")
        pos = torch.tensor([c[1] + i for c in chunks for i in range(len(c[0]))], dtype=torch.int64, device="cuda")
        seq = _i32([s for s, c in enumerate(chunks) for _ in c[0]])
        cu, slots = _cu([len(c[0]) for c in chunks]), _i32([c[2] for c in chunks])
        out = ops.embed_bigram_pos_f32(emb, ids, pos, big, (buckets, mp, mc), cu, seq, slots, prev, freq)
        ops.prev_token_update(prev, ids, cu, slots)
        return out.cpu()

    o1 = step([(a[:3], 0, 2), (b[:1], 0, 0)])
    o2 = step([(b[1:3], 1, 0), (a[3:4], 3, 2)])
    o3 = step([(a[4:], 4, 2)])
    o4 = step([(b, 0, 2)])                                    # b again, on the slot that a used
    got_a = torch.cat([o1[:3], o2[2:3], o3])
    got_b = torch.cat([o1[3:4], o2[:2]])
    tol = 2e-4                                                # angles in fp32: position 699 times a rounded frequency
    assert (got_a - ra).abs().max() < tol and (got_b - rb[:3]).abs().max() < tol and (o4 - rb).abs().max() < tol
    # without the table and without positions: the plain embedding
    plain = ops.embed_bigram_pos_f32(emb, torch.tensor(b, device="cuda"), torch.arange(len(b), device="cuda"))
    assert torch.equal(plain.cpu(), wt["embed"][b])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_relu_squared(dtype):
    from mi355_decode import ops
    for n in (1, 7, 4096, 5000):
        x = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 3).to(dtype)
        want = (torch.relu(x.float()) ** 2).to(dtype)
        assert torch.equal(ops.relu_squared(x.cuda()).cpu(), want)


def _paged(T, num_pages, seed):
    """A shuffled block table for one sequence of T tokens and its slot mapping."""
    order = np.random.default_rng(seed).permutation(num_pages)[: (T + 15) // 16].astype(np.int32)
    pos = np.arange(T)
    return order, order[pos // 16].astype(np.int64) * 16 + pos % 16


def _attn_in_cuts(q, k, wq, wk, r1, r2, gate, cuts, size, scale, eps=1e-5, pages=None, tiled=False, splits=0):
    """Norm + page write + attention over one sequence fed in portions through shuffled, NaN-filled
    pages; returns [T, H * d] float32."""
    from mi355_decode import ops
    T, H, d = q.shape
    G, dt = k.shape[1], q.dtype
    pages = pages or (T + 15) // 16 + 3
    table, slots = _paged(T, pages, 5)
    kc = torch.full((pages, G, 16, d), float("nan"), dtype=dt, device="cuda")
    vc = torch.full((pages, G, d, 16), float("nan"), dtype=dt, device="cuda")
    bt = torch.zeros(1, pages, dtype=torch.int32)
    bt[0, : len(table)] = torch.from_numpy(table)
    outs, at = [], 0
    for n in list(cuts) + [T]:
        n = min(n, T - at)
        if n == 0:
            break
        sl = slice(at, at + n)
        # one row holds q | k | gate, as the runner's fused projection does: column slices, not copies
        row = torch.cat([q[sl].reshape(n, -1), k[sl].reshape(n, -1), gate[sl]], dim=1).contiguous().cuda()
        qq, kk, gg = row[:, : H * d], row[:, H * d: (H + G) * d], row[:, (H + G) * d:]
        pos = torch.arange(at, at + n, dtype=torch.int64, device="cuda")
        ops.qk_norm_kv_write(qq, kk, kk, wq.cuda(), wk.cuda(), torch.from_numpy(slots[sl]).cuda(), kc, vc, H, G, d, d, eps)
        tiles = torch.from_numpy(ops.query_tiles([0, n])).cuda() if tiled else None
        out = ops.softmax_bias_attn(qq, kc, vc, bt.cuda(), torch.zeros(n, dtype=torch.int32, device="cuda"), pos, r1.cuda(),
                                    r2.cuda(), gg, H, scale, block=size, tiles=tiles, num_splits=splits if n <= 2 else 0)
        outs.append(out.float().cpu())
        at += n
    assert at == T
    return torch.cat(outs)


@pytest.mark.parametrize("H,G,d,size", [(6, 2, 16, 20), (3, 3, 24, 7), (2, 1, 32, 64), (4, 4, 20, 1), (4, 1, 8, 0), (1, 1, 136, 40),
                                        (8, 2, 64, 1000)])
def test_block_attention_whole_portions_and_single_tokens(H, G, d, size):
    g = torch.Generator().manual_seed(H * 100 + d)
    T = 75
    q, k = torch.randn(T, H, d, generator=g) * 2, torch.randn(T, G, d, generator=g) * 2
    wq, wk = torch.randn(d, generator=g) * 0.2 + 1, torch.randn(d, generator=g) * 0.2 + 1
    r1, r2 = torch.rand(H, generator=g) * 1.5, torch.rand(H, generator=g)
    gate = torch.randn(T, H * d, generator=g)
    ref = R.block_attention(q, k, wq, wk, r1, r2, 0.3, size, 1e-5, gate)
    for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
        got = _attn_in_cuts(q, k, wq, wk, r1, r2, gate, cuts, size, 0.3)
        assert (got - ref).abs().max() <= 3e-5 * ref.abs().max(), cuts
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    got = _attn_in_cuts(b16(q), b16(k), wq, wk, r1, r2, b16(gate), [40, 2, 1, 32], size, 0.3)
    ref = R.block_attention(b16(q).float(), b16(k).float(), wq, wk, r1, r2, 0.3, size, 1e-5, b16(gate).float())
    assert (got - ref).abs().max() <= 3e-2 * ref.abs().max()


@pytest.mark.parametrize("H,G,d,size", [(6, 2, 32, 20), (3, 3, 64, 7), (8, 2, 64, 48), (4, 4, 96, 1), (8, 1, 32, 0), (2, 1, 128, 40),
                                        (5, 1, 64, 33), (12, 2, 32, 17)])
def test_block_attention_on_the_matrix_cores(H, G, d, size):
    """bfloat16 inputs; the restatement sees the same rounded inputs, so what is left is the rounding of
    the stored pages, of the normed query and of the weights in the second product.  Single rows
    spread their keys over three workgroups."""
    g = torch.Generator().manual_seed(H * 100 + d)
    T = 75
    b16 = lambda t: t.to(torch.bfloat16)                      # noqa: E731
    q, k = b16(torch.randn(T, H, d, generator=g) * 2), b16(torch.randn(T, G, d, generator=g) * 2)
    wq, wk = torch.randn(d, generator=g) * 0.2 + 1, torch.randn(d, generator=g) * 0.2 + 1
    r1, r2 = torch.rand(H, generator=g) * 1.5, torch.rand(H, generator=g)
    gate = b16(torch.randn(T, H * d, generator=g))
    ref = R.block_attention(q.float(), k.float(), wq, wk, r1, r2, 0.3, size, 1e-5, gate.float())
    for cuts in ([T], [1] * T, [2, 3, 1, 30, 2, 16, 21]):
        got = _attn_in_cuts(q, k, wq, wk, r1, r2, gate, cuts, size, 0.3, tiled=True, splits=3)
        assert (got - ref).abs().max() <= 3e-2 * ref.abs().max(), cuts


@pytest.mark.parametrize("size", [16, 17, 31, 48, 64, 65, 400])
def test_block_edge_shows_with_one_loud_key(size):
    """The first token of the second block holds a key that every query scores far above all
    others, and a value unlike any other: queries see it exactly while they are in that block (for
    the widest block: one key among four hundred, two dozen pages back, against the distance
    penalty of head 1), and the last token of the first block never does."""
    H, G, d = 2, 1, 32
    j0, T = size, 2 * size + 6
    g = torch.Generator().manual_seed(size)
    q, k = torch.zeros(T, H, d), torch.randn(T, G, d, generator=g) * 0.1
    k[:, :, 3] = 0.0
    k[j0, 0] = 0.0
    k[j0, 0, 3] = 5.0                                         # normed: sqrt(32) on channel 3; as a value: 5 on channel 3
    q[:, :, 3] = 4.0                                          # normed: sqrt(32) on channel 3: score 32 * scale
    one = torch.ones(d)
    r1, r2 = torch.tensor([0.0, 0.5]), torch.tensor([0.0, 2.0])
    gate = torch.full((T, H * d), 20.0)                       # an open gate
    ref = R.block_attention(q, k, one, one, r1, r2, 1.0, size, 1e-5, gate)
    last_in, first_out = 2 * size - 1, 2 * size
    assert float(ref[last_in, 3]) > 4.9 and float(ref[last_in, d + 3]) > 4.9          # both heads, the far end of the block
    assert abs(float(ref[first_out, 3])) < 1e-3 and abs(float(ref[j0 - 1, 3])) < 1e-3  # the next block; the block before
    for cuts in ([T], [last_in, 1, 1] + [1] * 5, [5, 2] + [1] * (T - 7), [j0, 1, 2, 2]):
        got = _attn_in_cuts(q, k, one, one, r1, r2, gate, cuts, size, 1.0)
        assert (got - ref).abs().max() <= 1e-4 * ref.abs().max(), cuts
        b16 = lambda t: t.to(torch.bfloat16)                  # noqa: E731
        got = _attn_in_cuts(b16(q), b16(k), one, one, r1, r2, b16(gate), cuts, size, 1.0, tiled=True, splits=4)
        r16 = R.block_attention(b16(q).float(), b16(k).float(), one, one, r1, r2, 1.0, size, 1e-5, b16(gate).float())
        assert (got - r16).abs().max() <= 3e-2 * r16.abs().max(), cuts


def test_distance_penalty_moves_weight_to_near_keys():
    """All keys equal in score: without the penalty the output is the mean of the values, with it the
    weights fall as (1 + r2 distance)^(-r1)."""
    H, G, d, T = 2, 1, 16, 40
    q, k = torch.zeros(T, H, d), torch.zeros(T, G, d)
    k[:, 0, 0] = torch.arange(1, T + 1, dtype=torch.float32)           # the value's channel 0 names the position
    q[:, :, 1] = 1.0
    one = torch.ones(d)
    r1, r2 = torch.tensor([0.0, 2.0]), torch.tensor([0.0, 1.0])
    gate = torch.full((T, H * d), 30.0)
    got = _attn_in_cuts(q, k, one, one, r1, r2, gate, [17, 1, 1], 0, 1.0)
    w = (1.0 + torch.arange(T - 1, -1, -1, dtype=torch.float64)) ** -2.0
    want1 = float((w * torch.arange(1, T + 1, dtype=torch.float64)).sum() / w.sum())
    assert abs(float(got[-1, 0]) - (T + 1) / 2) < 1e-3 and abs(float(got[-1, d]) - want1) < 1e-3


def _gru_in_steps(x, bz, bx, C, chunks_per_step, state, parts=None):
    """x [T, 3 C + pad] rows of one or more sequences; chunks_per_step: [[(row slice, first position, slot)]]."""
    from mi355_decode import ops
    outs = {}
    for chunks in chunks_per_step:
        rows = torch.cat([x[c[0]] for c in chunks]).contiguous().cuda()
        pos = torch.cat([torch.arange(c[1], c[1] + (c[0].stop - c[0].start)) for c in chunks]).cuda()
        out = ops.mingru_scan(rows, 8, 8 + C, 8 + 2 * C, C, bz.cuda(), bx.cuda(), state, _cu([c[0].stop - c[0].start for c in chunks]),
                              pos, _i32([c[2] for c in chunks]), long_chunks=max(c[0].stop - c[0].start for c in chunks) > 1,
                              num_parts=parts)
        at = 0
        for c in chunks:
            n = c[0].stop - c[0].start
            outs.setdefault(c[2], []).append(out[at:at + n].float().cpu())
            at += n
    return {s: torch.cat(v) for s, v in outs.items()}


def _gru_ref(x, bz, bx, C):
    x = x.float()
    z = torch.sigmoid(x[:, 8:8 + C] + bz)
    c = R.mingru_candidate(x[:, 8 + C:8 + 2 * C] + bx)
    g = x[:, 8 + 2 * C:8 + 3 * C]
    return R.mingru_scan(z, c) * (g * torch.sigmoid(g))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [1, 33, 64, 200])
def test_mingru_whole_portions_single_tokens_and_long_prompts(dtype, C):
    g = torch.Generator().manual_seed(C)
    T = 1500 if C == 33 else 90                                # the long one: every wave of the workgroup scans many rows
    x = (torch.randn(T, 8 + 3 * C + 5, generator=g) * 2).to(dtype)
    bz, bx = torch.randn(C, generator=g), torch.randn(C, generator=g)
    ref = _gru_ref(x, bz, bx, C)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    state = torch.full((3, C), float("nan"), device="cuda")
    cuts_list = [[T], [2, 3, 1, 30, 2, 16, T - 54]] + ([[1] * T] if T < 200 else [[700, 1, 799]])
    for cuts in cuts_list:
        for parts in (None, 1, 3, 16):                         # a chunk dealt out to several workgroups, two launches
            steps, at = [], 0
            for n in cuts:
                steps.append([(slice(at, at + n), at, 1)])
                at += n
            got = _gru_in_steps(x, bz, bx, C, steps, state, parts)[1]
            assert (got - ref).abs().max() <= tol * ref.abs().max(), (cuts, parts)


def test_mingru_slots_are_separate_reset_at_position_zero_and_hold_a_value():
    C = 70
    g = torch.Generator().manual_seed(3)
    xa, xb = torch.randn(30, 8 + 3 * C, generator=g) * 2, torch.randn(20, 8 + 3 * C, generator=g) * 2
    # channel 5 of a: written at token 0 (gate open, candidate 7.5), then the gate stays shut for good
    xa[:, 8 + 5], xa[0, 8 + 5], xa[0, 8 + C + 5] = -40.0, 40.0, 7.0
    bz, bx = torch.zeros(C), torch.zeros(C)
    state = torch.full((3, C), float("nan"), device="cuda")
    x = torch.cat([xa, xb])
    A, B = lambda a, b: slice(a, b), lambda a, b: slice(30 + a, 30 + b)     # noqa: E731
    got = _gru_in_steps(x, bz, bx, C, [[(A(0, 17), 0, 2), (B(0, 1), 0, 0)],       # a portion beside a single first token
                                       [(A(17, 18), 17, 2), (B(1, 20), 1, 0)],    # a single token beside a portion
                                       [(A(18, 30), 18, 2)]], state)
    ra, rb = _gru_ref(xa, bz, bx, C), _gru_ref(xb, bz, bx, C)
    assert (got[2] - ra).abs().max() <= 2e-5 * ra.abs().max() and (got[0] - rb).abs().max() <= 2e-5 * rb.abs().max()
    gate = xa[:, 8 + 2 * C + 5]
    assert (got[2][:, 5] - 7.5 * gate * torch.sigmoid(gate)).abs().max() < 1e-4   # thirty tokens on, the state is what token 0 wrote
    again = _gru_in_steps(x, bz, bx, C, [[(B(0, 20), 0, 2)]], state)[2]            # b on the slot a used: position 0 resets it
    assert (again - rb).abs().max() <= 2e-5 * rb.abs().max()


def test_softmax_routing_groups_by_their_best_identity_outputs_and_scale():
    from mi355_decode import ops
    g = torch.Generator().manual_seed(2)
    for E, top, count, keep in ((8, 2, 2, 1), (14, 4, 2, 1), (12, 3, 4, 2), (6, 1, 6, 2), (16, 4, 1, 1), (9, 9, 3, 3), (64, 8, 8, 4),
                                (160, 20, 5, 3), (600, 6, 6, 2)):
        z = torch.randn(300, E + 3, generator=g) * 2           # three more columns ride in the rows: not router outputs
        # corrections that push every choice score below zero: a barred expert must not beat them as a "0"
        for corr in (torch.randn(E, generator=g) * 0.05, torch.randn(E, generator=g) * 0.05 - 3.0):
            ids, wts = ops.moe_route(z.cuda(), corr.cuda(), top, count, keep, softmax=True, group_max=True, weight_scale=1.5,
                                     experts=E)
            rid, rw = R.route(z[:, :E], corr, top, count, keep, 1.5)
            assert torch.equal(ids.cpu().long().sort(-1).values, rid.sort(-1).values), (E, top, count, keep)
            got = torch.zeros(300, E).scatter_(1, ids.cpu().long(), wts.cpu())
            want = torch.zeros(300, E).scatter_(1, rid, rw)
            assert (got - want).abs().max() < 1e-6
    # a group whose two best sum highest but whose best is not the highest: the two rules differ
    z = torch.log(torch.tensor([[0.30, 0.02, 0.02, 0.02, 0.22, 0.22, 0.10, 0.10]]))
    zero = torch.zeros(8)
    by_max, _ = ops.moe_route(z.cuda(), zero.cuda(), 2, 2, 1, softmax=True, group_max=True)
    by_two, _ = ops.moe_route(z.cuda(), zero.cuda(), 2, 2, 1, softmax=True, group_max=False)
    assert sorted(by_max.cpu().tolist()[0]) == [0, 1]
    assert sorted(by_two.cpu().tolist()[0]) == [4, 5]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 5, 300])
@pytest.mark.parametrize("W,F,S,identity", [(72, 40, 24, 3), (96, 64, 32, 0), (64, 16, 0, 2)])
def test_mixture_with_limits_identity_and_shared_experts(dtype, T, W, F, S, identity):
    """The mixture through the runner's feed-forward object: few rows take the per-row kernels, many
    rows library products per expert; inputs large enough that both limits bite."""
    from types import SimpleNamespace
    from mi355_decode.config import MoESpec
    from mi355_decode.hybrid_runner import MoEFeedForward
    g = torch.Generator().manual_seed(T + W)
    E, top, n = 6, 3, 6 + identity
    count = 3 if n % 3 == 0 else 2
    wt = {"router": torch.randn(n, W, generator=g) * W ** -0.5, "correction": torch.randn(n, generator=g) * 0.05}
    for name, ff in [(f"e{e}.", F) for e in range(E)] + ([("shared.", S)] if S else []):
        wt[name + "gate"], wt[name + "up"] = torch.randn(ff, W, generator=g) * W ** -0.5, torch.randn(ff, W, generator=g) * W ** -0.5
        wt[name + "down"] = torch.randn(W, ff, generator=g) * ff ** -0.5
    if S:
        wt["shared.sg"] = torch.randn(1, W, generator=g) * W ** -0.5
    wt = {k: v.to(torch.bfloat16).float() for k, v in wt.items()}
    h = (torch.randn(T, W, generator=g) * 2).to(dtype)
    mlp = {"expert": {"ff": F, "limit": 1.0}, "router": {"experts": E, "identity": identity, "top": top, "scale": 2.0,
                                                         "groups": {"count": count, "keep": 2}}}
    if S:
        mlp["shared"] = {"ff": S, "limit": 0.5}
    ref = R.moe_ff(wt, "", mlp, h.float())
    cat = lambda p: torch.cat([wt[p + "gate"], wt[p + "up"]])     # noqa: E731
    router = torch.cat([wt["router"]] + ([wt["shared.sg"]] if S else []))
    lw = SimpleNamespace(router_w=router.cuda(), correction=wt["correction"].cuda(),
                         gate_up_w=torch.stack([cat(f"e{e}.") for e in range(E)]).to(dtype).cuda(),
                         down_w=torch.stack([wt[f"e{e}.down"] for e in range(E)]).to(dtype).cuda(),
                         shared_gate_up_w=cat("shared.").to(dtype).cuda() if S else None,
                         shared_down_w=wt["shared.down"].to(dtype).cuda() if S else None)
    runner = SimpleNamespace(linear=lambda x, w: torch.mm(x, w.t()))
    spec = MoESpec(E, top, count, 2, F, score="softmax", group_score="max", weight_scale=2.0, identity=identity, limit=1.0,
                   shared_ff=S, shared_limit=0.5 if S else None)
    ff = MoEFeedForward(spec, lw, runner)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for min_rows, max_tokens in ((1, 2048), (1 << 30, 2048), (1, 64)):   # products per expert; the per-row kernels; in slices
        ff.GROUPED_MIN_ROWS, ff.GROUPED_MAX_TOKENS = min_rows, max_tokens
        got = ff(h.cuda()).float().cpu()
        assert (got - ref).abs().max() <= tol * ref.abs().max(), (min_rows, max_tokens)


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
        R.forward(_weights(name), CONFIGS[name], toks, trace=want)
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


@pytest.mark.parametrize("name", ["mix", "plain"])
def test_mixed_batches_equal_each_request_alone(name):
    """Four requests of unequal length advance together, portions beside single tokens; requests end and new
    ones take their pages and state slots."""
    eng = _engine(name, pages=24)
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
    for r in lens:
        _close(np.concatenate(got[r]), _ref(name, toks[r]))


def test_pages_and_slots_are_reused_without_leaking():
    eng = _engine("plain", pages=8, max_model_len=128)              # one 100-token request nearly fills the pool
    for i in range(6):
        toks = _tokens("plain", 100 - 7 * i, 50 + i)
        _close(_run_cuts(eng, f"r{i}", toks, [40, 3] + [1] * 10), _ref("plain", toks))


def test_long_decoding_past_blocks_and_pages():
    eng = _engine("mix")
    toks = _tokens("mix", 300, 9)
    _close(_run_cuts(eng, "long", toks, [10] + [1] * 290), _ref("mix", toks), tol=6e-4)


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
    run-ahead (the previous token of the hashed embedding travels in the state slot, on the
    device).  A token may leave the restatement's only where its own margin is inside the error."""
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
    args = ["--model", str(model_dir), "--served-model-name", "blocks", "--host", "127.0.0.1", "--port", str(port),
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
        post = lambda **body: client.http.post(f"{url}/v1/completions", json={"model": "blocks", **body})   # noqa: E731
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
