"""`bench.py --hybrid-compare`: hybrid (Lozupel) decoders at a few real layer sizes beside
Llama-shaped decoders of equal width, depth and parameter count, random weights.

Two parts.  (1) Through the engine: prompt tokens per second (a batch of prompts, chunked by the
scheduler) and decoded tokens per second (decode steps replayed from HIP graphs).  (2) Kernel by
kernel: the hybrid path's kernels timed alone at the prefill and the decode shape, each against
its own roofline (HBM bytes at 8 TB/s, bf16 MFMA at 2.5 PFLOP/s, or fp32 vector FMA at 157 TFLOP/s,
whichever bounds it), beside the like kernel of the Llama path at the same shape."""
from __future__ import annotations

import time

import numpy as np
import torch

from . import ops
from ._lib import BLOCK_SIZE
from .config import EngineArgs, ModelConfig

HBM, MFMA, VALU = 8.0e12, 2.5e15, 157.3e12


def tativik_config(width: int, layers: int, vocab: int = 32000) -> dict:
    """Alternating general-delta / latent-attention layers (every second attention reads the latent
    pages of the one before it), 64-wide recurrent heads, 128 + 64-wide attention heads over a latent of
    512, a 1024-token window, and in every layer 32 experts of width / 2 of which 4 run per token:
    as many active feed-forward weights as a dense feed-forward of 2 * width."""
    nh = width // 128
    ls, last_latent = [], None
    moe = {"kind": "moe", "expert": {"ff": width // 2},
           "router": {"experts": 32, "top": 4, "groups": {"count": 4, "keep": 2}}}
    for i in range(layers):
        if i % 2 == 0:
            ls.append({"type": "general_delta", "mixer": {"heads": width // 64, "dim": 64}, "mlp": moe})
            continue
        m = {"heads": nh, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": max(width * 3 // 8, 256),
             "mask": {"size": 1024}, "rot": {"dims": 64, "base": 1.0e6}, "scale": 192 ** -0.5}
        if last_latent is not None:
            m["kv_from"], last_latent = last_latent, None
        else:
            last_latent = i
        ls.append({"type": "latent_attention", "mixer": m, "mlp": moe})
    return {"architecture": "Tativik", "width": width, "vocab": vocab, "norm": {"eps": 1e-6, "groups": 4},
            "residual_mult": 0.7, "layers": ls}


def tafisun_config(width: int, layers: int, vocab: int = 32000) -> dict:
    """Alternating block-attention / minGRU layers: 128-wide heads, four query heads to a key head,
    blocks of 1024 positions; a recurrence as wide as the model; a dense relu^2 feed-forward of
    2 * width in the first layer and, in the others, 30 experts + 2 identity outputs of width / 2
    with 4 per token out of 2 of 4 groups, beside a shared expert of width / 2."""
    nh = width // 128
    att = {"heads": nh, "kv_heads": max(nh // 4, 1), "dim": 128, "vdim": 128, "mask": {"size": 1024}, "scale": 128 ** -0.5}
    moe = {"kind": "moe", "expert": {"ff": width // 2, "limit": 7.0}, "shared": {"ff": width // 2, "limit": 7.0},
           "router": {"experts": 30, "identity": 2, "top": 4, "scale": 1.5, "groups": {"count": 4, "keep": 2}}}
    ls = [{"type": "attention" if i % 2 == 0 else "mingru", "mixer": att if i % 2 == 0 else {"width": width},
           "mlp": {"kind": "dense", "ff": 2 * width} if i == 0 else moe} for i in range(layers)]
    return {"architecture": "Tafisun", "width": width, "vocab": vocab, "norm": {"eps": 1e-6},
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 1000003, "mul_cur": 7919}}, "layers": ls}


def bemulorn_config(width: int, layers: int, vocab: int = 32000, max_positions: int = 4096) -> dict:
    """Attention layers with parallel sub-layers: 128-wide heads, four query heads to a key head,
    chunks of 1024 positions, rotary positions on half of every head with blended frequencies; the
    second half of the layers reads the pages of the last layer of the first half; a limited gated
    feed-forward of 2 * width in the even layers and, in the odd ones, 32 experts of width / 2 with 4 per
    token beside a shared expert of width / 2."""
    nh = width // 128
    rot = {"dims": 64, "base": 10000.0, "scaling": {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}}
    att = {"heads": nh, "kv_heads": max(nh // 4, 1), "dim": 128, "vdim": 128, "mask": {"size": 1024}, "scale": 128 ** -0.5, "rot": rot}
    moe = {"kind": "moe", "expert": {"ff": width // 2}, "shared": {"ff": width // 2}, "router": {"experts": 32, "top": 4}}
    own = max(layers // 2, 1)
    ls = [{"type": "attention", "mixer": att if i < own else dict(att, kv_from=own - 1),
           "mlp": {"kind": "dense", "ff": 2 * width, "limit": 7.0} if i % 2 == 0 else moe} for i in range(layers)]
    return {"architecture": "Bemulorn", "width": width, "vocab": vocab, "max_positions": max_positions, "norm": {"eps": 1e-6},
            "embedding": {"scale": 2.0}, "logit_scale": 0.5, "layers": ls}


def lozupel_config(width: int, layers: int, vocab: int = 32000, loop: bool = True) -> dict:
    """Alternating parallel / delta layers with 128-wide heads, a 1024-token window, a feed-forward in
    every layer; the middle of the stack loops twice."""
    nh = width // 128
    left = {"heads": nh, "kv_heads": max(nh // 4, 1), "dim": 128, "vdim": 128, "mask": {"size": 1024},
            "rot": {"dims": 64, "base": 1.0e6}, "scale": 128 ** -0.5}
    right = {"heads": max(nh // 2, 1), "kv_heads": max(nh // 4, 1), "dim": 128, "vdim": 128, "conv": 4}
    delta = {"heads": nh, "kv_heads": max(nh // 2, 1), "dim": 128, "vdim": 128, "conv": 4}
    ff = {"kind": "dense", "ff": 2 * width}
    ls = [({"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": ff} if i % 2 == 0 else
           {"type": "delta", "mixer": delta, "mlp": ff}) for i in range(layers)]
    d = {"architecture": "Lozupel", "embedding": {"scale": 1.0}, "width": width, "vocab": vocab, "norm": {"eps": 1e-6},
         "logit_softcap": 30.0, "layers": ls}
    if layers >= 3 and loop:
        d["loop"] = {"start": 1, "stop": layers - 1, "times": 2}
    return d


def _params(weights) -> int:
    return sum(t.numel() for lw in weights.layers for t in (lw.tensors() if hasattr(lw, "tensors") else
                                                            (lw.qkv_w, lw.o_w, lw.gate_up_w, lw.down_w)))


def llama_config(width: int, layer_runs: int, layer_params: int, vocab: int = 32000) -> dict:
    """A Llama-shaped decoder of the same width and depth whose layers hold `layer_params` weights each."""
    nh, nkv, d = width // 128, max(width // 512, 1), 128
    attn = (nh + 2 * nkv) * d * width + nh * d * width
    inter = max(int((layer_params - attn) / (3 * width)) // 256 * 256, 256)
    return dict(architectures=["LlamaForCausalLM"], vocab_size=vocab, hidden_size=width, intermediate_size=inter,
                num_hidden_layers=layer_runs, num_attention_heads=nh, num_key_value_heads=nkv, rope_theta=1.0e6,
                rms_norm_eps=1e-6, max_position_embeddings=8192, tie_word_embeddings=False, torch_dtype="bfloat16")


def through_engine(cfg: ModelConfig, batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
    from .llm import build_engine
    from .sampling_params import SamplingParams
    eng = build_engine(EngineArgs(model="synthetic", dtype="bfloat16", max_num_seqs=batch,
                                  max_model_len=prompt_len + steps + warmup + 16, max_num_batched_tokens=8192,
                                  load_format="dummy", gpu_memory_utilization=0.9, seed=0), model_config=cfg)
    rng = np.random.default_rng(0)
    out = {"params_per_layer": _params(eng.runner.w) // max(len(eng.runner.w.layers), 1)}
    best = float("inf")
    pb = min(batch, 4)
    for rep in range(3):                                  # prompts: time from submission to every first token
        for i in range(pb):
            eng.add_request(f"p{rep}-{i}", rng.integers(0, cfg.vocab_size, prompt_len).tolist(),
                            SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.has_unfinished():
            eng.step()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
    out["prefill_tok_s"] = round(pb * prompt_len / best, 1)
    for i in range(batch):
        eng.add_request(f"d{i}", rng.integers(0, cfg.vocab_size, prompt_len).tolist(),
                        SamplingParams(max_tokens=warmup + steps + 8, temperature=0.0, ignore_eos=True))
    while eng.stats["decode_steps"] < warmup:
        eng.step()
    torch.cuda.synchronize()
    first, t0 = eng.stats["decode_steps"], time.perf_counter()
    while eng.stats["decode_steps"] < first + steps:
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    out["decode_ms_per_step"] = round(dt * 1e3 / steps, 4)
    out["decode_tok_s"] = round(batch * steps / dt, 1)
    out["decode_graphs"] = bool(eng.runner.graphs)
    for rid in list(eng.seqs):
        eng.abort_request(rid)
    while eng._pending:
        eng._harvest_decode()
    del eng
    torch.cuda.empty_cache()
    return out


def _time(fn, reps: int = 20) -> float:
    """Seconds per call: best of three event-timed runs of `reps` back-to-back launches."""
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        e.synchronize()
        best = min(best, s.elapsed_time(e) * 1e-3 / reps)
    return best


def kernel_table(width: int, prompt_len: int, batch: int) -> list:
    """[{kernel, shape, us, bound, frac_of_roofline, like, like_us, like_frac}]"""
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *s, dt=bf: torch.randn(*s, device=dev, dtype=torch.float32, generator=g).to(dt)  # noqa: E731
    H, G, d, dv, window = width // 128, max(width // 512, 1), 128, 128, 1024
    F = 2 * width
    rows = []

    def row(kernel, shape, t, bound, work, like=None, like_t=None, like_work=None):
        peak = {"hbm": HBM, "mfma": MFMA, "valu": VALU}[bound]
        r = {"kernel": kernel, "shape": shape, "us": round(t * 1e6, 2), "bound": bound,
             "frac_of_roofline": round(work / peak / t, 4)}
        if like is not None:
            r.update(like=like, like_us=round(like_t * 1e6, 2), like_frac=round(like_work / peak / like_t, 4))
        rows.append(r)

    for T, tag in ((prompt_len, "prefill"), (batch, "decode")):
        shape = f"{tag} {T} rows x {width}"
        resid, add16, w1, wv = rnd(T, width, dt=torch.float32), rnd(T, width), rnd(1), rnd(width)
        x16, r16, out16 = rnd(T, width), rnd(T, width), torch.empty(T, width, device=dev, dtype=bf)
        row("add_rms_norm_f32 (one-number weight)", shape, _time(lambda: ops.add_rms_norm_f32(resid, w1, 1e-6, add=add16, out=out16)),
            "hbm", T * width * 12, "fused_add_rms_norm", _time(lambda: ops.fused_add_rms_norm(x16, r16, wv, 1e-6, out=out16)),
            T * width * 8)
        xa, xb = rnd(T, width), rnd(T, width)
        row("rms_norm_mix_f32", shape, _time(lambda: ops.rms_norm_mix_f32(resid, xa, wv, xb, wv, 1e-6, 0.5)), "hbm",
            T * width * 12)
        gu, act = rnd(T, 2 * F), torch.empty(T, F, device=dev, dtype=bf)
        row("gelu_tanh_and_mul", f"{tag} {T} rows x {F}", _time(lambda: ops.gelu_tanh_and_mul(gu, out=act)), "hbm", T * F * 6,
            "silu_and_mul", _time(lambda: ops.silu_and_mul(gu, out=act)), T * F * 6)

    # ---- attention: one prompt of prompt_len tokens; then `batch` sequences decoding at that context
    P = prompt_len
    pages = (P + BLOCK_SIZE) // BLOCK_SIZE + 1
    nb = pages * batch
    kc, vct = rnd(nb, G, BLOCK_SIZE, d), rnd(nb, G, dv, BLOCK_SIZE)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(batch, pages)
    temp, bias = torch.ones(H, device=dev), torch.full((H,), -2.0, device=dev)
    q, gate = rnd(P, H * d), rnd(P, H)
    pos = torch.arange(P, dtype=torch.int64, device=dev)
    seq0 = torch.zeros(P, dtype=torch.int32, device=dev)
    cu, ctx = torch.tensor([0, P], dtype=torch.int32, device=dev), torch.tensor([P], dtype=torch.int32, device=dev)
    o = torch.empty(P, H * dv, device=dev, dtype=bf)
    keys = sum(min(i + 1, window) for i in range(P))
    tiles = torch.from_numpy(ops.query_tiles([0, P])).to(dev)
    nsp = max(min(16, 2048 // max(tiles.shape[0] * G * max(H // G // 4, 1), 1)), 1)
    ppart = torch.empty(nsp * P * H * dv, device=dev)
    t_h = _time(lambda: ops.sigmoid_window_attn(q, kc, vct, bt[:1], seq0, pos, temp, bias, gate, H, window, d ** -0.5, out=o,
                                                tiles=tiles, partial=ppart, num_splits=nsp), 5)
    t_l = _time(lambda: ops.paged_attn_prefill(q, kc, vct, bt[:1], cu, ctx, P, H, G, d, d ** -0.5, out=o), 5)
    row("sigmoid_window_attn", f"prefill {P} tokens, window {window}, {H}/{G} heads x {d}", t_h, "mfma", 2.0 * keys * H * (d + dv),
        "paged_attn_prefill (causal softmax)", t_l, 2.0 * (P * (P + 1) // 2) * H * 2 * d)
    qd, gd = rnd(batch, H * d), rnd(batch, H)
    posd = torch.full((batch,), P - 1, dtype=torch.int64, device=dev)
    seqd = torch.arange(batch, dtype=torch.int32, device=dev)
    ctxd = torch.full((batch,), P, dtype=torch.int32, device=dev)
    od = torch.empty(batch, H * dv, device=dev, dtype=bf)
    ws = torch.empty(max(ops.decode_workspace_bytes(batch, H, d, 16), 16), dtype=torch.uint8, device=dev)
    dtiles = torch.stack([seqd, seqd, torch.ones_like(seqd)], dim=1).contiguous()
    part = torch.empty(16 * batch * H * dv, device=dev)
    t_h = _time(lambda: ops.sigmoid_window_attn(qd, kc, vct, bt, seqd, posd, temp, bias, gd, H, window, d ** -0.5, out=od,
                                                tiles=dtiles, partial=part, num_splits=16))
    t_l = _time(lambda: ops.paged_attn_decode(qd, kc, vct, bt, ctxd, H, G, d, d ** -0.5, num_splits=4, workspace=ws, out=od))
    row("sigmoid_window_attn", f"decode {batch} rows at context {P}, window {window}", t_h, "hbm",
        batch * min(P, window) * G * (d + dv) * 2, "paged_attn_decode (whole context)", t_l, batch * P * G * 2 * d * 2)

    # ---- the recurrence: heads of 128 x 128 state
    Hd, Gd = width // 128, max(width // 256, 1)
    C = 2 * Gd * d + Hd * dv
    for T, S, tag in ((P, 1, "prefill"), (batch, batch, "decode")):
        x = rnd(T, C)
        conv_w = rnd(C, 4)
        cst = torch.zeros(S + 1, 3, C, device=dev)
        st = torch.zeros(S + 1, Hd, d, dv, device=dev)
        per = T // S
        cu_ = torch.arange(0, T + 1, per, dtype=torch.int32, device=dev)
        pos_ = (torch.arange(T, device=dev) % per + (0 if S == 1 else P)).to(torch.int64)
        seq_ = (torch.arange(T, device=dev) // per).to(torch.int32)
        slots = torch.arange(S, dtype=torch.int32, device=dev)
        y = torch.empty(T, C, device=dev, dtype=bf)
        row("causal_conv_silu + state update", f"{tag} {T} rows x {C} channels, 4 taps",
            _time(lambda: ops.causal_conv_silu(x, conv_w, cst, seq_, pos_, cu_, slots, out=y)), "hbm", T * C * 4)
        beta, dec = rnd(T, Hd), rnd(T, Hd)
        a_log, dtb = torch.zeros(Hd, device=dev), torch.zeros(Hd, device=dev)
        oo = torch.empty(T, Hd, dv, device=dev)
        t = _time(lambda: ops.gated_delta_rule(x, 0, Gd * d, 2 * Gd * d, beta, dec, a_log, dtb, st, cu_, pos_, slots, Hd, Gd, d,
                                               dv, out=oo, long_chunks=S == 1), 5)
        if S == 1:
            row("gated_delta_rule", f"prefill {T} tokens, {Hd} heads x {d} x {dv}", t, "valu", 6.0 * T * Hd * d * dv)
        else:
            row("gated_delta_rule", f"decode {S} rows, {Hd} heads x {d} x {dv}", t, "hbm", S * Hd * d * dv * 8)
        gt, hn = rnd(T, Hd * dv), torch.ones(dv, device=dev)
        on = torch.empty(T, Hd * dv, device=dev, dtype=bf)
        row("gated_head_rms_norm", f"{tag} {T} rows x {Hd} heads x {dv}", _time(lambda: ops.gated_head_rms_norm(oo, gt, hn, 1e-6, 0, out=on)),
            "hbm", T * Hd * dv * 8)
    return rows


def compare(widths, layers: int, batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
    result = {"metric": "hybrid_vs_llama_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "config": {"layers": layers, "batch": batch, "prompt_len": prompt_len, "decode_steps": steps},
              "models": [], "kernels": {}}
    for width in widths:
        hc = ModelConfig.from_dict(lozupel_config(width, layers))
        h = through_engine(hc, batch, prompt_len, steps, warmup)
        runs = len(hc.hybrid.runs())
        # equal size: as many layer runs, as many weights read per run
        lc = ModelConfig.from_dict(llama_config(width, runs, h["params_per_layer"]))
        ll = through_engine(lc, batch, prompt_len, steps, warmup)
        result["models"].append({"width": width, "layer_runs": runs, "hybrid": h, "llama": ll,
                                 "prefill_ratio": round(h["prefill_tok_s"] / ll["prefill_tok_s"], 3),
                                 "decode_ratio": round(h["decode_tok_s"] / ll["decode_tok_s"], 3)})
        result["kernels"][str(width)] = kernel_table(width, prompt_len, batch)
    return result


def tativik_kernel_table(width: int, prompt_len: int, batch: int) -> list:
    """The sandwich arrangement's kernels at the prefill and the decode shape, each against its own
    roofline, beside the like kernel of the "pre" arrangement (the Lozupel design) at the same shape."""
    from types import SimpleNamespace
    from .config import MoESpec
    from .hybrid_runner import MoEFeedForward, rotary_table
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *s, dt=bf: torch.randn(*s, device=dev, dtype=torch.float32, generator=g).to(dt)  # noqa: E731
    rows = []

    def row(kernel, shape, t, bound, work, like=None, like_t=None, like_work=None, like_bound=None):
        peak = {"hbm": HBM, "mfma": MFMA, "valu": VALU}
        r = {"kernel": kernel, "shape": shape, "us": round(t * 1e6, 2), "bound": bound,
             "frac_of_roofline": round(work / peak[bound] / t, 4)}
        if like is not None:
            r.update(like=like, like_us=round(like_t * 1e6, 2), like_frac=round(like_work / peak[like_bound or bound] / like_t, 4))
            r["distance_ratio"] = round(r["like_frac"] / max(r["frac_of_roofline"], 1e-9), 2)
        rows.append(r)

    P, W = prompt_len, width
    for T, tag in ((P, "prefill"), (batch, "decode")):
        shape = f"{tag} {T} rows x {W}"
        resid, add16, w1 = rnd(T, W, dt=torch.float32), rnd(T, W), rnd(1)
        wv32, b32, out16 = rnd(W, dt=torch.float32), rnd(W, dt=torch.float32), torch.empty(T, W, device=dev, dtype=bf)
        row("group_rms_norm_f32 (4 groups)", shape, _time(lambda: ops.group_rms_norm_f32(resid, wv32, 4, 1e-6, dtype=bf, out=out16)),
            "hbm", T * W * 6, "add_rms_norm_f32", _time(lambda: ops.add_rms_norm_f32(resid, w1, 1e-6, out=out16)), T * W * 6)
        y, gate, wv = rnd(T, W), rnd(T, W), rnd(W)
        row("gated_norm_resid_f32 (4 groups)", shape,
            _time(lambda: ops.gated_norm_resid_f32(resid, y, gate, b32, wv32, 4, 1e-6, 0.7)), "hbm", T * W * 12,
            "rms_norm_mix_f32 (two inputs)", _time(lambda: ops.rms_norm_mix_f32(resid, y, wv, gate, wv, 1e-6, 0.5)), T * W * 12)

    # ---- attention: one prompt of P tokens; then `batch` sequences decoding at that context
    H, R_, rot, window = W // 128, 512, 64, 1024
    G, d, dv = max(W // 512, 1), 128, 128
    pages = (P + BLOCK_SIZE) // BLOCK_SIZE + 1
    nb = pages * batch
    cache, cache_t = rnd(nb, BLOCK_SIZE, R_ + rot), rnd(nb, R_, BLOCK_SIZE)
    kc, vct = rnd(nb, G, BLOCK_SIZE, d), rnd(nb, G, dv, BLOCK_SIZE)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(batch, pages)
    cs = rotary_table(rot, 1.0e6, pages * BLOCK_SIZE, dev)
    sink, temp, bias = torch.zeros(H, device=dev), torch.ones(H, device=dev), torch.full((H,), -2.0, device=dev)
    keys = sum(min(i + 1, window) for i in range(P))
    for T, tag in ((P, "prefill"), (batch, "decode")):
        ql, q, gt = rnd(H, T, R_) * 0.05, rnd(T, H * (128 + rot)), rnd(T, H)
        qs = rnd(T, H * d)
        if tag == "prefill":
            pos, seq, b_t = torch.arange(P, dtype=torch.int64, device=dev), torch.zeros(P, dtype=torch.int32, device=dev), bt[:1]
            tiles = torch.from_numpy(ops.query_tiles([0, P])).to(dev)
            nsp = max(min(16, 2048 // max(tiles.shape[0] * G * max(H // G // 4, 1), 1)), 1)
            nkeys, shape = keys, f"prefill {P} tokens, window {window}"
        else:
            pos, seq, b_t = torch.full((T,), P - 1, dtype=torch.int64, device=dev), torch.arange(T, dtype=torch.int32, device=dev), bt
            tiles = torch.stack([seq, seq, torch.ones_like(seq)], dim=1).contiguous()
            nsp, nkeys, shape = 16, T * min(P, window), f"decode {T} rows at context {P}, window {window}"
        part = torch.empty(nsp * T * H * dv, device=dev)
        ol, o = torch.empty(H, T, R_, device=dev, dtype=bf), torch.empty(T, H * dv, device=dev, dtype=bf)
        cu_h = [0, P] if tag == "prefill" else list(range(T + 1))
        ptiles = torch.from_numpy(ops.pair_tiles(cu_h, H)).to(dev)
        qe = ops.latent_q_pack(ql, q, 128 + rot, 128, rot, cs, pos)
        nspl = min(16, max(window // 64, 1), max(1024 // int(ptiles.shape[0]), 1))
        t_n = _time(lambda: ops.latent_window_attn_tiles(qe, cache, cache_t, b_t, ptiles, pos, sink, gt, window, 0.07,
                                                         num_splits=nspl, out=ol), 5)
        t_l = _time(lambda: ops.sigmoid_window_attn(qs, kc, vct, b_t, seq, pos, temp, bias, gt, H, window, d ** -0.5, out=o,
                                                    tiles=tiles, partial=part, num_splits=nsp), 5)
        if tag == "prefill":
            row("latent_window_attn", f"{shape}, {H} heads x ({R_} + {rot})", t_n, "mfma", 2.0 * nkeys * H * (2 * R_ + rot),
                f"sigmoid_window_attn, {H}/{G} heads x {d}", t_l, 2.0 * nkeys * H * (d + dv))
        else:
            row("latent_window_attn", f"{shape}, {H} heads x ({R_} + {rot})", t_n, "hbm", nkeys * (R_ + rot) * 2,
                f"sigmoid_window_attn, {H}/{G} heads x {d}", t_l, nkeys * G * (d + dv) * 2)
        x, nw = rnd(T, R_ + rot), torch.ones(R_, device=dev)
        slots = (torch.arange(T, device=dev) if tag == "prefill" else torch.arange(T, device=dev) * pages * BLOCK_SIZE + P - 1).to(torch.int64)
        k_, v_ = rnd(T, G * d), rnd(T, G * dv)
        cs2 = rotary_table(64, 1.0e6, pages * BLOCK_SIZE, dev)
        row("latent_kv_write (norm + rotation)", f"{tag} {T} rows x {R_ + rot}",
            _time(lambda: ops.latent_kv_write(x, nw, cs, pos, slots, cache, R_, rot, 1e-6, cache_t=cache_t)), "hbm",
            T * (3 * R_ + 2 * rot) * 2,
            "rope_partial_kv_write", _time(lambda: ops.rope_partial_kv_write(qs, k_, v_, cs2, pos, slots, kc, vct, H, G, d, dv)),
            T * (2 * H * d + 2 * G * (d + dv)) * 2)

    # ---- the recurrences: heads of 64 x 64 state beside the gated rule's 128 x 128, equal state per layer
    Hn, dn = W // 64, 64
    Hd, Gd, dd = W // 128, max(W // 256, 1), 128
    for T, S, tag in ((P, 1, "prefill"), (batch, batch, "decode")):
        per = T // S
        cu_ = torch.arange(0, T + 1, per, dtype=torch.int32, device=dev)
        pos_ = (torch.arange(T, device=dev) % per + (0 if S == 1 else P)).to(torch.int64)
        slots = torch.arange(S, dtype=torch.int32, device=dev)
        xn = rnd(T, 5 * Hn * dn)
        C = Hn * dn
        w0, ab = torch.zeros(C, device=dev), torch.zeros(C, device=dev)
        stn = torch.zeros(S + 1, Hn, dn, dn, device=dev)
        on = torch.empty(T, Hn, dn, device=dev)
        t_n = _time(lambda: ops.general_delta_rule(xn[:, :C], xn[:, C:2 * C], xn[:, 2 * C:3 * C], xn[:, 3 * C:4 * C], w0,
                                                   xn[:, 4 * C:], ab, stn, cu_, pos_, slots, Hn, dn, out=on, long_chunks=S == 1), 5)
        Cd = 2 * Gd * dd + Hd * dd
        xd, beta, dec = rnd(T, Cd), rnd(T, Hd), rnd(T, Hd)
        a_log, dtb = torch.zeros(Hd, device=dev), torch.zeros(Hd, device=dev)
        std = torch.zeros(S + 1, Hd, dd, dd, device=dev)
        od = torch.empty(T, Hd, dd, device=dev)
        t_l = _time(lambda: ops.gated_delta_rule(xd, 0, Gd * dd, 2 * Gd * dd, beta, dec, a_log, dtb, std, cu_, pos_, slots, Hd,
                                                 Gd, dd, dd, out=od, long_chunks=S == 1), 5)
        if S == 1:
            row("general_delta_rule", f"prefill {T} tokens, {Hn} heads x {dn} x {dn}", t_n, "valu", 8.0 * T * Hn * dn * dn,
                f"gated_delta_rule, {Hd} heads x {dd} x {dd}", t_l, 6.0 * T * Hd * dd * dd)
        else:
            row("general_delta_rule", f"decode {S} rows, {Hn} heads x {dn} x {dn}", t_n, "hbm", S * Hn * dn * dn * 8,
                f"gated_delta_rule, {Hd} heads x {dd} x {dd}", t_l, S * Hd * dd * dd * 8)

    # ---- the mixture of experts beside a dense gated feed-forward with as many active weights
    E, top, F = 32, 4, W // 2
    lw = SimpleNamespace(router_w=rnd(E, W, dt=torch.float32) * W ** -0.5, correction=torch.zeros(E, device=dev),
                         gate_up_w=rnd(E, 2 * F, W) * W ** -0.5, down_w=rnd(E, W, F) * F ** -0.5)
    ff = MoEFeedForward(MoESpec(E, top, 4, 2, F), lw, None)
    gu_w, dn_w = rnd(2 * top * F, W) * W ** -0.5, rnd(W, top * F) * F ** -0.5
    for T, tag in ((P, "prefill"), (batch, "decode")):
        h = rnd(T, W)
        t_n = _time(lambda: ff(h), 5)
        if tag == "prefill":
            dense = lambda: torch.mm(ops.gelu_tanh_and_mul(torch.mm(h, gu_w.t())), dn_w.t())   # noqa: E731
            row("mixture of experts (route, sort, expert GEMMs, sum)", f"prefill {T} rows, {top} of {E} experts x {F}", t_n,
                "mfma", 6.0 * T * top * F * W, "dense gated feed-forward (library GEMMs)", _time(dense, 5), 6.0 * T * top * F * W)
        else:
            dense = lambda: ops.linear_decode(ops.gelu_tanh_and_mul(ops.linear_decode(h, gu_w)), dn_w)   # noqa: E731
            touched = min(E, T * top)
            row("mixture of experts (route, sort, per-row products, sum)", f"decode {T} rows, {top} of {E} experts x {F}", t_n,
                "hbm", touched * 3 * F * W * 2, "dense gated feed-forward (weight stream)", _time(dense, 5), 3 * top * F * W * 2)
    return rows


def compare_tativik(widths, layers: int, batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
    """The sandwich arrangement (Tativik) beside the closest existing model, the "pre" arrangement
    (Lozupel), at equal width and depth and as many active feed-forward weights."""
    result = {"metric": "tativik_vs_lozupel_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "config": {"layers": layers, "batch": batch, "prompt_len": prompt_len, "decode_steps": steps},
              "models": [], "kernels": {}}
    for width in widths:
        t = through_engine(ModelConfig.from_dict(tativik_config(width, layers)), batch, prompt_len, steps, warmup)
        z = through_engine(ModelConfig.from_dict(lozupel_config(width, layers, loop=False)), batch, prompt_len, steps, warmup)
        result["models"].append({"width": width, "layers": layers, "tativik": t, "lozupel": z,
                                 "prefill_ratio": round(t["prefill_tok_s"] / z["prefill_tok_s"], 3),
                                 "decode_ratio": round(t["decode_tok_s"] / z["decode_tok_s"], 3)})
        result["kernels"][str(width)] = tativik_kernel_table(width, prompt_len, batch)
    return result


def tafisun_kernel_table(width: int, prompt_len: int, batch: int) -> list:
    """The Tafisun design's kernels at the prefill and the decode shape, each against its own
    roofline, beside the like kernel of the closest existing designs at the same shape."""
    from types import SimpleNamespace
    from .config import MoESpec
    from .hybrid_runner import MoEFeedForward
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *s, dt=bf: torch.randn(*s, device=dev, dtype=torch.float32, generator=g).to(dt)  # noqa: E731
    rows = []

    def row(kernel, shape, t, bound, work, like=None, like_t=None, like_work=None, like_bound=None):
        peak = {"hbm": HBM, "mfma": MFMA, "valu": VALU}
        r = {"kernel": kernel, "shape": shape, "us": round(t * 1e6, 2), "bound": bound,
             "frac_of_roofline": round(work / peak[bound] / t, 4)}
        if like is not None:
            r.update(like=like, like_us=round(like_t * 1e6, 2), like_frac=round(like_work / peak[like_bound or bound] / like_t, 4))
            r["distance_ratio"] = round(r["like_frac"] / max(r["frac_of_roofline"], 1e-9), 2)
        rows.append(r)

    P, W, V = prompt_len, width, 32000
    H, G, d, block = W // 128, max(W // 512, 1), 128, 1024
    pages = (P + BLOCK_SIZE) // BLOCK_SIZE + 1
    nb = pages * batch
    kc, vct = rnd(nb, G, BLOCK_SIZE, d), rnd(nb, G, d, BLOCK_SIZE)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(batch, pages)
    embed, bigram = rnd(V, W), rnd(65522, W)
    freq = torch.from_numpy((10000.0 ** (-2.0 * np.arange(W // 2) / W)).astype(np.float32)).to(dev)
    r1, r2 = torch.full((H,), 0.5, device=dev), torch.full((H,), 0.3, device=dev)
    temp, bias = torch.ones(H, device=dev), torch.full((H,), -2.0, device=dev)
    wn = torch.ones(d, device=dev)
    cs = None
    for T, S, tag in ((P, 1, "prefill"), (batch, batch, "decode")):
        shape = f"{tag} {T} rows x {W}"
        per = T // S
        cu = torch.arange(0, T + 1, per, dtype=torch.int32, device=dev)
        pos = (torch.arange(T, device=dev) % per + (0 if S == 1 else P - 1)).to(torch.int64)
        seq = (torch.arange(T, device=dev) // per).to(torch.int32)
        slots = torch.arange(S, dtype=torch.int32, device=dev)
        ids = torch.randint(0, V, (T,), device=dev, generator=g)
        prev = torch.zeros(S + 1, dtype=torch.int32, device=dev)
        # ---- embedding
        row("embed_bigram_pos_f32 + prev_token_update", shape,
            _time(lambda: (ops.embed_bigram_pos_f32(embed, ids, pos, bigram, (65521, 1000003, 7919), cu, seq, slots, prev, freq),
                           ops.prev_token_update(prev, ids, cu, slots))), "hbm", T * W * 8,
            "embed_scale_f32", _time(lambda: ops.embed_scale_f32(embed, ids, 1.0)), T * W * 6)
        # ---- feed-forward activation
        F = 2 * W
        up, gu, act = rnd(T, F), rnd(T, 2 * F), torch.empty(T, F, device=dev, dtype=bf)
        row("relu_squared", f"{tag} {T} rows x {F}", _time(lambda: ops.relu_squared(up)), "hbm", T * F * 4,
            "gelu_tanh_and_mul", _time(lambda: ops.gelu_tanh_and_mul(gu, out=act)), T * F * 6)
        # ---- attention
        if cs is None:
            from .hybrid_runner import rotary_table
            cs = rotary_table(64, 1.0e6, pages * BLOCK_SIZE, dev)
        proj = rnd(T, (2 * H + G) * d)
        q, k, gt = proj[:, : H * d], proj[:, H * d: (H + G) * d], proj[:, (H + G) * d:]
        v_, gh = rnd(T, G * d), rnd(T, H)
        wslots = (torch.arange(T, device=dev) if S == 1 else torch.arange(T, device=dev) * pages * BLOCK_SIZE + P - 1).to(torch.int64)
        row("qk_norm_kv_write", f"{tag} {T} rows, {H}/{G} heads x {d}",
            _time(lambda: ops.qk_norm_kv_write(q, k, k, wn, wn, wslots, kc, vct, H, G, d, d, 1e-6)), "hbm",
            T * (2 * H * d + 3 * G * d) * 2,
            "rope_partial_kv_write", _time(lambda: ops.rope_partial_kv_write(q, k, v_, cs, pos, wslots, kc, vct, H, G, d, d)),
            T * (2 * H * d + 4 * G * d) * 2)
        if S == 1:
            tiles = torch.from_numpy(ops.query_tiles([0, P])).to(dev)
            b_t = bt[:1]
        else:
            tiles = torch.stack([seq, seq, torch.ones_like(seq)], dim=1).contiguous()
            b_t = bt
        rep = H // G
        hb = 4 if rep % 4 == 0 else 3 if rep % 3 == 0 else 2 if rep % 2 == 0 else 1
        nsb = max(min(16, block // 64, 1024 // max(int(tiles.shape[0]) * G * (rep // hb), 1)), 1)
        nsw = max(min(16, 2048 // max(int(tiles.shape[0]) * G * max(rep // 4, 1), 1)), 1)
        part = torch.empty(nsw * T * H * d, device=dev)
        o = torch.empty(T, H * d, device=dev, dtype=bf)
        t_n = _time(lambda: ops.softmax_bias_attn(q, kc, vct, b_t, seq, pos, r1, r2, gt, H, d ** -0.5, block=block, tiles=tiles,
                                                  num_splits=nsb if nsb > 1 else 0), 5)
        t_l = _time(lambda: ops.sigmoid_window_attn(q, kc, vct, b_t, seq, pos, temp, bias, gh, H, block, d ** -0.5, out=o,
                                                    tiles=tiles, partial=part, num_splits=nsw), 5)
        if S == 1:
            keys_b = sum(i % block + 1 for i in range(P))
            keys_w = sum(min(i + 1, block) for i in range(P))
            row("softmax_bias_attn", f"prefill {P} tokens, blocks of {block}, {H}/{G} heads x {d}", t_n, "mfma",
                2.0 * keys_b * H * 2 * d, f"sigmoid_window_attn, window {block}", t_l, 2.0 * keys_w * H * 2 * d)
        else:
            kb = (P - 1) % block + 1
            row("softmax_bias_attn", f"decode {T} rows at position {P - 1}: {kb} keys each, blocks of {block}", t_n, "hbm",
                T * kb * G * 2 * d * 2, f"sigmoid_window_attn, window {block}: {min(P, block)} keys each", t_l,
                T * min(P, block) * G * 2 * d * 2)
        # ---- the recurrence
        C = W
        x3 = rnd(T, 3 * C)
        bz, bx = torch.zeros(C, device=dev), torch.zeros(C, device=dev)
        st = torch.zeros(S + 1, C, device=dev)
        t_n = _time(lambda: ops.mingru_scan(x3, 0, C, 2 * C, C, bz, bx, st, cu, pos, slots, long_chunks=S == 1), 5)
        Hd, Gd, dd = W // 128, max(W // 256, 1), 128
        Cd = 2 * Gd * dd + Hd * dd
        xd, beta, dec = rnd(T, Cd), rnd(T, Hd), rnd(T, Hd)
        a_log, dtb = torch.zeros(Hd, device=dev), torch.zeros(Hd, device=dev)
        std = torch.zeros(S + 1, Hd, dd, dd, device=dev)
        od = torch.empty(T, Hd, dd, device=dev)
        t_l = _time(lambda: ops.gated_delta_rule(xd, 0, Gd * dd, 2 * Gd * dd, beta, dec, a_log, dtb, std, cu, pos, slots, Hd, Gd, dd,
                                                 dd, out=od, long_chunks=S == 1), 5)
        if S == 1:
            row("mingru_scan", f"prefill {T} tokens x {C} channels", t_n, "hbm", T * C * 8,
                f"gated_delta_rule, {Hd} heads x {dd} x {dd}", t_l, 6.0 * T * Hd * dd * dd, "valu")
        else:
            row("mingru_scan", f"decode {S} rows x {C} channels", t_n, "hbm", S * C * 16,
                f"gated_delta_rule, {Hd} heads x {dd} x {dd}", t_l, S * Hd * dd * dd * 8)
    # ---- the mixture of experts beside the sigmoid-routed one without identity and shared experts
    E, I, top, F = 30, 2, 4, W // 2
    lw = SimpleNamespace(router_w=rnd(E + I + 1, W, dt=torch.float32) * W ** -0.5, correction=torch.zeros(E + I, device=dev),
                         gate_up_w=rnd(E, 2 * F, W) * W ** -0.5, down_w=rnd(E, W, F) * F ** -0.5,
                         shared_gate_up_w=rnd(2 * F, W) * W ** -0.5, shared_down_w=rnd(W, F) * F ** -0.5)
    lin = SimpleNamespace(linear=lambda x, w: ops.linear_decode(x, w) if x.shape[0] <= ops.LINEAR_DECODE_MAX_M else torch.mm(x, w.t()))
    ff = MoEFeedForward(MoESpec(E, top, 4, 2, F, score="softmax", group_score="max", weight_scale=1.5, identity=I, limit=7.0,
                                shared_ff=F, shared_limit=7.0), lw, lin)
    lw0 = SimpleNamespace(router_w=rnd(E + I, W, dt=torch.float32) * W ** -0.5, correction=torch.zeros(E + I, device=dev),
                          gate_up_w=rnd(E + I, 2 * F, W) * W ** -0.5, down_w=rnd(E + I, W, F) * F ** -0.5)
    ff0 = MoEFeedForward(MoESpec(E + I, top, 4, 2, F), lw0, None)
    for T, tag in ((P, "prefill"), (batch, "decode")):
        h = rnd(T, W)
        t_n, t_l = _time(lambda: ff(h), 5), _time(lambda: ff0(h), 5)
        if tag == "prefill":
            row("mixture (softmax route, identity, limits, shared expert)", f"prefill {T} rows, {top} of {E}+{I} x {F}, shared {F}", t_n,
                "mfma", 6.0 * T * (top + 1) * F * W, "mixture (sigmoid route), no shared expert", t_l, 6.0 * T * top * F * W)
        else:
            touched = min(E, T * top)
            row("mixture (softmax route, identity, limits, shared expert)", f"decode {T} rows, {top} of {E}+{I} x {F}, shared {F}", t_n,
                "hbm", (touched + 1) * 3 * F * W * 2, "mixture (sigmoid route), no shared expert", t_l,
                min(E + I, T * top) * 3 * F * W * 2)
    return rows


def compare_tafisun(widths, layers: int, batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
    """The Tafisun design beside the closest existing model, the sandwich arrangement (Tativik: a
    softmax attention in a window, a recurrence, a grouped mixture of experts), at equal width and depth."""
    result = {"metric": "tafisun_vs_tativik_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "config": {"layers": layers, "batch": batch, "prompt_len": prompt_len, "decode_steps": steps},
              "models": [], "kernels": {}}
    for width in widths:
        t = through_engine(ModelConfig.from_dict(tafisun_config(width, layers)), batch, prompt_len, steps, warmup)
        z = through_engine(ModelConfig.from_dict(tativik_config(width, layers)), batch, prompt_len, steps, warmup)
        result["models"].append({"width": width, "layers": layers, "tafisun": t, "tativik": z,
                                 "prefill_ratio": round(t["prefill_tok_s"] / z["prefill_tok_s"], 3),
                                 "decode_ratio": round(t["decode_tok_s"] / z["decode_tok_s"], 3)})
        result["kernels"][str(width)] = tafisun_kernel_table(width, prompt_len, batch)
    return result


def bemulorn_kernel_table(width: int, prompt_len: int, batch: int) -> list:
    """The Bemulorn design's kernels at the prefill and the decode shape, each against its own
    roofline, beside the like kernel of the closest existing paths (the Llama-shaped decoder's for
    attention, norm and activation; the Tafisun design's mixture) at the same shape."""
    from types import SimpleNamespace
    from .config import MoESpec, RotaryScaling
    from .hybrid_runner import MoEFeedForward, rotary_table
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *s, dt=bf: torch.randn(*s, device=dev, dtype=torch.float32, generator=g).to(dt)  # noqa: E731
    rows = []

    def row(kernel, shape, t, bound, work, like=None, like_t=None, like_work=None, like_bound=None):
        peak = {"hbm": HBM, "mfma": MFMA, "valu": VALU}
        r = {"kernel": kernel, "shape": shape, "us": round(t * 1e6, 2), "bound": bound,
             "frac_of_roofline": round(work / peak[bound] / t, 4)}
        if like is not None:
            r.update(like=like, like_us=round(like_t * 1e6, 2), like_frac=round(like_work / peak[like_bound or bound] / like_t, 4))
            r["distance_ratio"] = round(r["like_frac"] / max(r["frac_of_roofline"], 1e-9), 2)
        rows.append(r)

    P, W, V = prompt_len, width, 32000
    H, G, d, chunk = W // 128, max(W // 512, 1), 128, 1024
    pages = (P + BLOCK_SIZE) // BLOCK_SIZE + 1
    nb = pages * batch
    kc, vct = rnd(nb, G, BLOCK_SIZE, d), rnd(nb, G, d, BLOCK_SIZE)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(batch, pages)
    embed, ptab = rnd(V, W), rnd(pages * BLOCK_SIZE, W)
    sink = torch.zeros(H, device=dev)
    cs = rotary_table(64, 10000.0, pages * BLOCK_SIZE, dev, RotaryScaling(4.0, 1024.0, 32.0, 1.0))
    F = 2 * W
    for T, S, tag in ((P, 1, "prefill"), (batch, batch, "decode")):
        shape = f"{tag} {T} rows x {W}"
        per = T // S
        pos = (torch.arange(T, device=dev) % per + (0 if S == 1 else P - 1)).to(torch.int64)
        seq = (torch.arange(T, device=dev) // per).to(torch.int32)
        ids = torch.randint(0, V, (T,), device=dev, generator=g)
        # ---- embedding
        row("embed_scale_pos_f32", shape, _time(lambda: ops.embed_scale_pos_f32(embed, ids, 2.0, ptab, pos)), "hbm", T * W * 8,
            "embed_scale_f32", _time(lambda: ops.embed_scale_f32(embed, ids, 2.0)), T * W * 6)
        # ---- the one norm of a layer, the previous layer's output riding in its launch
        resid, add16, wv = rnd(T, W, dt=torch.float32), rnd(T, W), rnd(W)
        x16, r16, out16 = rnd(T, W), rnd(T, W), torch.empty(T, W, device=dev, dtype=bf)
        row("add_rms_norm_f32 (vector weight)", shape, _time(lambda: ops.add_rms_norm_f32(resid, wv, 1e-6, add=add16, out=out16)),
            "hbm", T * W * 12, "fused_add_rms_norm", _time(lambda: ops.fused_add_rms_norm(x16, r16, wv, 1e-6, out=out16)), T * W * 8)
        # ---- the gated activation: column slices of the fused projection into a slice of the output row
        proj = rnd(T, (H + 2 * G) * d + 8 + 2 * F)
        at = (H + 2 * G) * d + 8
        rowbuf = torch.empty(T, H * d + F, device=dev, dtype=bf)
        gu, act = rnd(T, 2 * F), torch.empty(T, F, device=dev, dtype=bf)
        row("gated_act_rows (limited unit, column slices)", f"{tag} {T} rows x {F}",
            _time(lambda: ops.gated_act_rows(proj[:, at: at + F], proj[:, at + F: at + 2 * F], 7.0, out=rowbuf[:, H * d:])), "hbm",
            T * F * 6, "silu_and_mul", _time(lambda: ops.silu_and_mul(gu, out=act)), T * F * 6)
        # ---- rotation and page write
        q, k, v_ = proj[:, : H * d], proj[:, H * d: (H + G) * d], proj[:, (H + G) * d: (H + 2 * G) * d]
        gh = proj[:, (H + 2 * G) * d: (H + 2 * G) * d + H]
        wslots = (torch.arange(T, device=dev) if S == 1 else torch.arange(T, device=dev) * pages * BLOCK_SIZE + P - 1).to(torch.int64)
        wn = torch.ones(d, device=dev)
        row("rope_partial_kv_write (64 of 128 rotated)", f"{tag} {T} rows, {H}/{G} heads x {d}",
            _time(lambda: ops.rope_partial_kv_write(q, k, v_, cs, pos, wslots, kc, vct, H, G, d, d)), "hbm",
            T * (2 * H * d + 4 * G * d) * 2,
            "qk_norm_kv_write", _time(lambda: ops.qk_norm_kv_write(q, k, k, wn, wn, wslots, kc, vct, H, G, d, d, 1e-6)),
            T * (2 * H * d + 3 * G * d) * 2)
        row("rope_partial_kv_write (queries alone: shared pages)", f"{tag} {T} rows, {H} heads x {d}",
            _time(lambda: ops.rope_partial_kv_write(q, None, None, cs, pos, wslots, None, None, H, G, d, d)), "hbm",
            T * 2 * H * d * 2)
        # ---- attention beside the Llama path's
        if S == 1:
            tiles = torch.from_numpy(ops.query_tiles([0, P])).to(dev)
            b_t = bt[:1]
        else:
            tiles = torch.stack([seq, seq, torch.ones_like(seq)], dim=1).contiguous()
            b_t = bt
        rep = H // G
        hb = 4 if rep % 4 == 0 else 3 if rep % 3 == 0 else 2 if rep % 2 == 0 else 1
        nsb = max(min(16, chunk // 64, 1024 // max(int(tiles.shape[0]) * G * (rep // hb), 1)), 1)
        out_slice = rowbuf[:, : H * d]
        t_n = _time(lambda: ops.softmax_bias_attn(q, kc, vct, b_t, seq, pos, None, None, gh, H, d ** -0.5, block=chunk, tiles=tiles,
                                                  num_splits=nsb if nsb > 1 else 0, sink=sink, out=out_slice), 5)
        o = torch.empty(T, H * d, device=dev, dtype=bf)
        qc = q.contiguous()
        if S == 1:
            cu, ctx = torch.tensor([0, P], dtype=torch.int32, device=dev), torch.tensor([P], dtype=torch.int32, device=dev)
            t_l = _time(lambda: ops.paged_attn_prefill(qc, kc, vct, bt[:1], cu, ctx, P, H, G, d, d ** -0.5, out=o), 5)
            keys_b = sum(i % chunk + 1 for i in range(P))
            # what the runner takes for prompts at these sizes: the LDS-staged form
            t_s = _time(lambda: ops.paged_attn_prefill_ext(q, kc, vct, bt[:1], cu, ctx, P, H, G, d, d ** -0.5, chunk=chunk, sink=sink,
                                                           gate=gh, out=out_slice), 5)
            row("paged_attn_prefill_ext (chunks, value-less term, head gates)", f"prefill {P} tokens, chunks of {chunk}, {H}/{G} heads x {d}",
                t_s, "mfma", 2.0 * keys_b * H * 2 * d, "paged_attn_prefill (causal softmax)", t_l, 2.0 * (P * (P + 1) // 2) * H * 2 * d)
            row("softmax_bias_attn, tile form (prompts of other head sizes)", f"prefill {P} tokens, chunks of {chunk}, {H}/{G} heads x {d}", t_n,
                "mfma", 2.0 * keys_b * H * 2 * d, "paged_attn_prefill (causal softmax)", t_l, 2.0 * (P * (P + 1) // 2) * H * 2 * d)
        else:
            ctxd = torch.full((batch,), P, dtype=torch.int32, device=dev)
            ws = torch.empty(max(ops.decode_workspace_bytes(batch, H, d, 16), 16), dtype=torch.uint8, device=dev)
            t_l = _time(lambda: ops.paged_attn_decode(qc, kc, vct, bt, ctxd, H, G, d, d ** -0.5, num_splits=4, workspace=ws, out=o))
            kb = (P - 1) % chunk + 1
            row("softmax_bias_attn (value-less term, head gates)", f"decode {T} rows at position {P - 1}: {kb} keys each, chunks of {chunk}",
                t_n, "hbm", T * kb * G * 2 * d * 2, f"paged_attn_decode (whole context: {P} keys each)", t_l, T * P * G * 2 * d * 2)
    # ---- the mixture (choice by logits, softmax over the chosen, biased router; the shared expert's rows come
    # ---- from the layer's output product) beside the Tafisun design's (softmax route in groups, identity and
    # ---- shared experts)
    E, top, Fe = 32, 4, W // 2
    lw = SimpleNamespace(router_w=rnd(E, W, dt=torch.float32) * W ** -0.5, router_b=torch.zeros(E, device=dev),
                         correction=torch.zeros(E, device=dev), gate_up_w=rnd(E, 2 * Fe, W) * W ** -0.5,
                         down_w=rnd(E, W, Fe) * Fe ** -0.5)
    ff = MoEFeedForward(MoESpec(E, top, 1, 1, Fe, score="chosen_softmax", router_bias=True, shared_gated=False), lw, None)
    lin = SimpleNamespace(linear=lambda x, w: ops.linear_decode(x, w) if x.shape[0] <= ops.LINEAR_DECODE_MAX_M else torch.mm(x, w.t()))
    lw0 = SimpleNamespace(router_w=rnd(E + 1, W, dt=torch.float32) * W ** -0.5, correction=torch.zeros(E, device=dev),
                          gate_up_w=rnd(E - 2, 2 * Fe, W) * W ** -0.5, down_w=rnd(E - 2, W, Fe) * Fe ** -0.5,
                          shared_gate_up_w=rnd(2 * Fe, W) * W ** -0.5, shared_down_w=rnd(W, Fe) * Fe ** -0.5)
    ff0 = MoEFeedForward(MoESpec(E - 2, top, 4, 2, Fe, score="softmax", group_score="max", weight_scale=1.5, identity=2, limit=7.0,
                                 shared_ff=Fe, shared_limit=7.0), lw0, lin)
    for T, tag in ((P, "prefill"), (batch, "decode")):
        h, other = rnd(T, W), rnd(T, W)
        t_n, t_l = _time(lambda: ff(h, shared=other), 5), _time(lambda: ff0(h), 5)
        if tag == "prefill":
            row("mixture (choice by logits, softmax over the chosen)", f"prefill {T} rows, {top} of {E} x {Fe}", t_n, "mfma",
                6.0 * T * top * Fe * W, "mixture (softmax route in groups, identity, limits, shared expert)", t_l,
                6.0 * T * (top + 1) * Fe * W)
        else:
            row("mixture (choice by logits, softmax over the chosen)", f"decode {T} rows, {top} of {E} x {Fe}", t_n, "hbm",
                min(E, T * top) * 3 * Fe * W * 2, "mixture (softmax route in groups, identity, limits, shared expert)", t_l,
                (min(E - 2, T * top) + 1) * 3 * Fe * W * 2)
    return rows


def compare_bemulorn(widths, layers: int, batch: int, prompt_len: int, steps: int, warmup: int) -> dict:
    """The Bemulorn design beside the closest existing model, a Llama-shaped decoder (rotary
    grouped-query softmax attention, gated feed-forward) of equal width, depth and weights per layer."""
    result = {"metric": "bemulorn_vs_llama_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "config": {"layers": layers, "batch": batch, "prompt_len": prompt_len, "decode_steps": steps},
              "models": [], "kernels": {}}
    for width in widths:
        bc = ModelConfig.from_dict(bemulorn_config(width, layers, max_positions=prompt_len + steps + warmup + 16))
        b = through_engine(bc, batch, prompt_len, steps, warmup)
        lc = ModelConfig.from_dict(llama_config(width, layers, b["params_per_layer"]))
        ll = through_engine(lc, batch, prompt_len, steps, warmup)
        result["models"].append({"width": width, "layers": layers, "bemulorn": b, "llama": ll,
                                 "prefill_ratio": round(b["prefill_tok_s"] / ll["prefill_tok_s"], 3),
                                 "decode_ratio": round(b["decode_tok_s"] / ll["decode_tok_s"], 3)})
        result["kernels"][str(width)] = bemulorn_kernel_table(width, prompt_len, batch)
    return result
