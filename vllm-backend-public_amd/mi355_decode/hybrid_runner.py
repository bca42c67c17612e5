"""One model step on one GPU for hybrid decoders (config.HybridSpec): every layer names its sequence
mixer and may carry a feed-forward.  Two arrangements share this runner:
  * "pre" (the Lozupel design): a gated delta rule (a linear recurrence with a matrix state per
    head), or a sliding-window attention with sigmoid weights beside such a recurrence, and a dense
    gated feed-forward; a span of layers can run several times with shared weights;
    a third design of this arrangement (Tafisun) adds a hashed previous-token embedding and
    sinusoidal positions to the embedding, and mixes by a softmax attention inside blocks of positions
    (logarithmic distance penalty, keys as values, normed queries and keys, a gate per output channel)
    or by a per-channel gated recurrence; its feed-forward is relu^2 or a softmax-routed mixture with
    identity experts and a shared expert;
  * "sandwich" (the Tativik design): a general delta rule (decay per key channel, removal along the
    unit key) or a softmax attention through low-rank latents (sliding window, a sink in the
    denominator, latent pages that a later layer may share), then a mixture of experts; every
    sub-layer sits between a norm in groups and a gated, normed, scaled residual add;
  * "parallel" (the Bemulorn design): one norm per layer whose output both sub-layers read,
    x += attention(h) + ff(h); learned positions beside a scaled embedding; the attention is the
    block attention without norms and penalty but with biased projections, rotary positions on part
    of every head (frequencies blended for long contexts), a value-less term in the softmax
    denominator, one gate per head and key / value pages that a later layer may share; the
    feed-forward is a limited gated unit or a mixture whose weights are a softmax over the chosen
    logits, plus an ungated shared expert.

What differs from ModelRunner's decoders, and where it lives:
  * the residual stream is float32 (csrc/resid32.hip: norms with one learned number or a vector,
    residual adds, the gelu-tanh gate, the logit soft cap); activations and weights are bfloat16
    (or float32 throughout with dtype float32: every kernel here is built for both);
  * K/V pages hold rotated keys [blocks, kv_heads, 16, dim] and values [blocks, kv_heads, vdim, 16],
    one pair per layer RUN (a looped layer has one per pass), on the engine's block tables;
  * recurrent and convolution state lives in per-sequence slots (engine.SlotAllocator), again one
    set per layer run; a chunk that starts at position 0 resets its slot;
  * one step function, `_forward`, serves prompts, portions of prompts and decoded tokens in one
    packed batch (csrc/seqmix.hip).  run_prefill drives it eagerly; the decode step drives the same
    function from the static step inputs and is captured into a HIP graph per batch bucket.

Shares ModelRunner's step machinery: static step inputs and pinned staging, graph capture and
replay, run-ahead, sampling, log-probabilities.  One GPU only.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from . import ops
from ._lib import BLOCK_SIZE
from .config import ModelConfig
from .model_runner import ModelRunner, batch_buckets
from .weights import ModelWeights


def rotary_table(rot_dims: int, base: float, max_pos: int, device, scaling=None) -> torch.Tensor:
    """float32 [max_pos, rot_dims] = cos | sin of pos * base^(-2i / rot_dims), i < rot_dims / 2.
    scaling (config.RotaryScaling): its blended frequencies instead, cos and sin times its factor.
    Angles are formed in float32 from float32 frequencies."""
    half = rot_dims // 2
    mult = 1.0
    if scaling is None:
        inv = float(base) ** (-2.0 * torch.arange(half, dtype=torch.float32, device=device) / rot_dims)
    else:
        f, mult = scaling.frequencies(rot_dims, base)
        inv = torch.from_numpy(f.astype(np.float32)).to(device)
    ang = torch.arange(max_pos, dtype=torch.float32, device=device)[:, None] * inv[None, :]
    return (torch.cat([ang.cos(), ang.sin()], dim=1) * mult).contiguous()


class StepBatch:
    """Device-side description of one packed step (see csrc/seqmix.hip)."""
    __slots__ = ("ids", "positions", "slot_mapping", "block_tables", "cu_seqlens", "tok_seq", "state_slots",
                 "num_tokens", "num_seqs", "tiles", "long_chunks", "pair_tiles", "context_lens", "max_q_len")

    def __init__(self, ids, positions, slot_mapping, block_tables, cu_seqlens, tok_seq, state_slots, tiles=None,
                 long_chunks=False, pair_tiles=None, context_lens=None, max_q_len=0):
        # every chunk's length of context after the step (int32, on the device) and the longest chunk: what the
        # LDS-staged prompt attention walks by; None: not known to this step (captured decode steps)
        self.context_lens, self.max_q_len = context_lens, int(max_q_len)
        self.tiles = tiles                            # 16-row query tiles (ops.query_tiles) or None: one wave per row
        self.pair_tiles = pair_tiles                  # heads -> tiles of 16 (row, head) pairs (ops.pair_tiles), or None
        self.long_chunks = long_chunks                # some chunk holds several tokens (prompts and portions)
        self.ids, self.positions, self.slot_mapping, self.block_tables = ids, positions, slot_mapping, block_tables
        self.cu_seqlens, self.tok_seq, self.state_slots = cu_seqlens, tok_seq, state_slots
        self.num_tokens, self.num_seqs = int(ids.numel()), int(cu_seqlens.numel()) - 1


class WindowAttention:
    """Sliding-window attention with sigmoid weights over the paged K/V of one layer run."""

    def __init__(self, spec, lw, runner, cache_index: int):
        self.s, self.lw, self.r, self.ci = spec, lw, runner, cache_index

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        s, seg, r = self.s, self.lw.seg, self.r
        q = proj[:, seg["lq"][0]: seg["lq"][0] + seg["lq"][1]]
        k = proj[:, seg["lk"][0]: seg["lk"][0] + seg["lk"][1]]
        v = proj[:, seg["lv"][0]: seg["lv"][0] + seg["lv"][1]]
        g = proj[:, seg["lg"][0]: seg["lg"][0] + seg["lg"][1]]
        kc, vc = r.k_cache[self.ci], r.v_cache[self.ci]
        ops.rope_partial_kv_write(q, k, v, r.rotary(s.rot_dims, s.rot_base), b.positions, b.slot_mapping, kc, vc,
                                  s.heads, s.kv_heads, s.dim, s.vdim)
        o = ops.sigmoid_window_attn(q, kc, vc, b.block_tables, b.tok_seq, b.positions, self.lw.attn_temp,
                                    self.lw.attn_bias, g, s.heads, s.window, s.scale, tiles=b.tiles,
                                    **r.key_splits(b, s))
        return r.linear(o, self.lw.attn_o_w)


class DeltaMixer:
    """Gated delta rule with its convolution, decay, gate and output norm, on one layer run's state slots."""

    def __init__(self, spec, lw, runner, state_index: int):
        self.s, self.lw, self.r, self.si = spec, lw, runner, state_index

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        s, lw, seg, r = self.s, self.lw, self.lw.seg, self.r
        qk, vv = s.kv_heads * s.dim, s.heads * s.vdim
        q0 = seg["q"][0]
        if seg["k"][0] != q0 + qk or seg["v"][0] != q0 + 2 * qk:
            raise RuntimeError("q | k | v of a delta mixer must be adjacent in the input projection")
        conv_state, rec_state = r.conv_state[self.si], r.rec_state[self.si]
        y = ops.causal_conv_silu(proj[:, q0: q0 + 2 * qk + vv], lw.conv_w, conv_state, b.tok_seq, b.positions,
                                 b.cu_seqlens, b.state_slots)
        beta = proj[:, seg["b"][0]: seg["b"][0] + s.heads]
        if s.per_channel:
            decay = r.linear(proj[:, seg["a1"][0]: seg["a1"][0] + seg["a1"][1]], lw.a2_w)
            gate = r.linear(proj[:, seg["g1"][0]: seg["g1"][0] + seg["g1"][1]], lw.g2_w)
        else:
            decay = proj[:, seg["a"][0]: seg["a"][0] + s.heads]
            gate = proj[:, seg["g"][0]: seg["g"][0] + vv]
        o = ops.gated_delta_rule(y, 0, qk, 2 * qk, beta, decay, lw.a_log, lw.dt_bias, rec_state, b.cu_seqlens,
                                 b.positions, b.state_slots, s.heads, s.kv_heads, s.dim, s.vdim,
                                 per_channel=s.per_channel, long_chunks=b.long_chunks)
        on = ops.gated_head_rms_norm(o, gate, lw.head_norm, r.eps, ops.ACT_SIGMOID if s.per_channel else ops.ACT_SILU)
        return r.linear(on, lw.delta_o_w)


class GeneralDeltaMixer:
    """General delta rule with its low-rank decay, removal rate, per-head output norm and gate, on one
    layer run's state slots."""

    def __init__(self, spec, lw, runner, state_index: int):
        self.s, self.lw, self.r, self.si = spec, lw, runner, state_index

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        s, lw, r = self.s, self.lw, self.r
        col = lambda n: proj[:, lw.seg[n][0]: lw.seg[n][0] + lw.seg[n][1]]     # noqa: E731
        decay = r.linear(ops.tanh_rows(col("w1")), lw.w2_w)
        o = ops.general_delta_rule(col("r"), col("k"), col("v"), decay, lw.w0, col("a"), lw.a_b, r.rec_state[self.si],
                                   b.cu_seqlens, b.positions, b.state_slots, s.heads, s.dim, long_chunks=b.long_chunks)
        return r.linear(ops.gated_head_rms_norm(o, col("g"), lw.head_norm, r.eps, ops.ACT_SIGMOID), lw.o_w)


class LatentAttention:
    """Sliding-window softmax attention through low-rank latents over the latent pages of one layer
    run -- its own (it writes them first) or those of the layer it shares with."""

    def __init__(self, spec, lw, runner, cache_index: int, writes: bool):
        self.s, self.lw, self.r, self.ci, self.writes = spec, lw, runner, cache_index, writes

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        s, lw, r = self.s, self.lw, self.r
        col = lambda n: proj[:, lw.seg[n][0]: lw.seg[n][0] + lw.seg[n][1]]     # noqa: E731
        (cache, cache_t), table = r.latent_cache[self.ci], r.rotary(s.rot_dims, s.rot_base)
        if self.writes:
            ops.latent_kv_write(col("dkv"), lw.dkv_norm, table, b.positions, b.slot_mapping, cache, s.kv_rank, s.rot_dim,
                                r.eps, cache_t=cache_t)
        q = r.linear(ops.rms_norm_rows(col("dq"), lw.dq_norm, r.eps), lw.uq_w)
        T, hw = q.shape[0], s.dim + s.rot_dim
        # the unrotated query part of every head into the latent space: the keys then are the cached latents
        ql = torch.bmm(q.view(T, s.heads, hw)[:, :, : s.dim].transpose(0, 1), lw.uk_w)
        if cache_t is not None and b.pair_tiles is not None:
            # the matrix cores: tiles of 16 (row, head) pairs; few tiles (decoded tokens, short prompts) spread
            # their windows' keys over several workgroups
            tiles = b.pair_tiles(s.heads)
            n = min(16, max(s.window // 64, 1), max(1024 // max(int(tiles.shape[0]), 1), 1))
            ol = ops.latent_window_attn_tiles(ops.latent_q_pack(ql, q, hw, s.dim, s.rot_dim, table, b.positions), cache,
                                              cache_t, b.block_tables, tiles, b.positions, lw.sink, col("g"), s.window,
                                              s.scale, num_splits=n)
        else:
            ol = ops.latent_window_attn(ql, q, hw, s.dim, cache, b.block_tables, b.tok_seq, b.positions, lw.sink, col("g"),
                                        table, s.window, s.scale)
        o = torch.bmm(ol, lw.uv_t)                      # [heads, tokens, vdim]
        return r.linear(o.transpose(0, 1).reshape(T, s.heads * s.vdim), lw.o_w)


class BlockAttention:
    """Softmax attention inside blocks of positions with a logarithmic distance penalty over the paged
    K/V of one layer run.  Queries and keys are RMS-normed per head; the V pages hold the keys as
    projected (the design has no value projection)."""

    def __init__(self, spec, lw, runner, cache_index: int):
        self.s, self.lw, self.r, self.ci = spec, lw, runner, cache_index

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        s, lw, r = self.s, self.lw, self.r
        col = lambda n: proj[:, lw.seg[n][0]: lw.seg[n][0] + lw.seg[n][1]]     # noqa: E731
        q, k = col("q"), col("k")
        kc, vc = r.k_cache[self.ci], r.v_cache[self.ci]
        ops.qk_norm_kv_write(q, k, k, lw.q_norm, lw.k_norm, b.slot_mapping, kc, vc, s.heads, s.kv_heads, s.dim, s.vdim, r.eps)
        o = ops.softmax_bias_attn(q, kc, vc, b.block_tables, b.tok_seq, b.positions, lw.r1, lw.r2, col("g"), s.heads,
                                  s.scale, block=s.block, tiles=b.tiles, num_splits=r.block_key_splits(b, s))
        return r.linear(o, lw.o_w)


class RotaryBlockAttention:
    """Softmax attention inside blocks of positions over the paged K/V of one layer run -- its own
    (it writes them first) or those of the layer it shares with: biased projections, rotary positions
    on the first rot_dims coordinates of every head, one more value-less term in the softmax
    denominator, one sigmoid gate per head.  Writes the gated heads into `out`, a column slice of
    the row that the layer's output matrix multiplies.  Steps that hold a portion of a prompt take the
    LDS-staged launch where the sizes allow (ops.chunk_attn_prefill_ok), all others the tile form."""

    def __init__(self, spec, lw, runner, cache_index: int, writes: bool):
        self.s, self.lw, self.r, self.ci, self.writes = spec, lw, runner, cache_index, writes

    def __call__(self, proj: torch.Tensor, b: StepBatch, out: torch.Tensor) -> torch.Tensor:
        s, lw, r = self.s, self.lw, self.r
        col = lambda n: proj[:, lw.seg[n][0]: lw.seg[n][0] + lw.seg[n][1]]     # noqa: E731
        q = col("q")
        kc, vc = r.k_cache[self.ci], r.v_cache[self.ci]
        table = r.rotary(s.rot_dims, s.rot_base, s.rot_scaling)
        if self.writes:
            ops.rope_partial_kv_write(q, col("k"), col("v"), table, b.positions, b.slot_mapping, kc, vc, s.heads, s.kv_heads,
                                      s.dim, s.vdim)
        elif s.rot_dims > 0:
            ops.rope_partial_kv_write(q, None, None, table, b.positions, b.slot_mapping, None, None, s.heads, s.kv_heads,
                                      s.dim, s.vdim)
        if b.long_chunks and b.context_lens is not None and ops.chunk_attn_prefill_ok(q.dtype, s.heads, s.kv_heads, s.dim, s.vdim) \
                and proj.stride(0) % 8 == 0 and out.stride(0) % 8 == 0:
            # prompts and portions (single tokens beside them ride along): K/V steps staged through LDS once for a
            # workgroup's tile of queries
            return ops.paged_attn_prefill_ext(q, kc, vc, b.block_tables, b.cu_seqlens, b.context_lens, b.max_q_len, s.heads,
                                              s.kv_heads, s.dim, s.scale, chunk=s.block, sink=lw.sink, gate=col("g"), out=out)
        return ops.softmax_bias_attn(q, kc, vc, b.block_tables, b.tok_seq, b.positions, None, None, col("g"), s.heads, s.scale,
                                     block=s.block, tiles=b.tiles, num_splits=r.block_key_splits(b, s), sink=lw.sink, out=out)


class MinGRUMixer:
    """Per-channel gated recurrence on one layer run's state slots: gates and candidate from the
    current token only, the state in float32."""

    def __init__(self, spec, lw, runner, state_index: int):
        self.s, self.lw, self.r, self.si = spec, lw, runner, state_index

    def __call__(self, proj: torch.Tensor, b: StepBatch) -> torch.Tensor:
        lw, seg = self.lw, self.lw.seg
        o = ops.mingru_scan(proj, seg["z"][0], seg["x"][0], seg["g"][0], self.s.width, lw.z_b, lw.x_b,
                            self.r.rec_state[self.si], b.cu_seqlens, b.positions, b.state_slots, long_chunks=b.long_chunks)
        return self.r.linear(o, lw.o_w)


class ReluSquaredFF:
    """Dense feed-forward without a gate: down(relu(up h)^2)."""

    def __init__(self, lw, runner):
        self.lw, self.r = lw, runner

    def __call__(self, h: torch.Tensor) -> torch.Tensor:
        return self.r.linear(ops.relu_squared(self.r.linear(h, self.lw.up_w)), self.lw.down_w)


class MoEFeedForward:
    """Mixture of experts: fp32 routing, rows sorted by expert, the expert products, the weighted sum
    (which also takes in identity experts and a gated shared expert where the design has them)."""

    GROUPED_MIN_ROWS = 512          # from this many routed rows on, one library GEMM per expert (needs the counts on the host)

    def __init__(self, spec, lw, runner):
        self.s, self.lw, self.r = spec, lw, runner

    GROUPED_MAX_TOKENS = 2048       # longer steps go through the experts in slices of this many tokens

    def __call__(self, h: torch.Tensor, shared: Optional[torch.Tensor] = None) -> torch.Tensor:
        """h [tokens, width] -> the mixture's output, the same shape.  Tokens are independent of each other
        here, so a long step is served in slices: the padded batched products then stay at sizes where
        an uneven slice costs little padding, and their temporaries at a few hundred megabytes.
        shared [tokens, width]: rows the caller has computed already (a shared expert, another
        sub-layer's output) that the weighted sum takes in unscaled, instead of a shared expert run here."""
        T = h.shape[0]
        if T <= self.GROUPED_MAX_TOKENS:
            return self._tokens(h, shared)
        out = torch.empty_like(h)
        for a in range(0, T, self.GROUPED_MAX_TOKENS):
            out[a: a + self.GROUPED_MAX_TOKENS] = self._tokens(h[a: a + self.GROUPED_MAX_TOKENS],
                                                               None if shared is None else shared[a: a + self.GROUPED_MAX_TOKENS])
        return out

    def _act(self, gu: torch.Tensor, limit, ff: int) -> torch.Tensor:
        if limit is None and gu.dtype != torch.float32 and ff % 8 == 0:
            return ops.silu_and_mul(gu)
        return ops.moe_silu_and_mul(gu, limit)

    def _tokens(self, h: torch.Tensor, shared: Optional[torch.Tensor] = None) -> torch.Tensor:
        s, lw = self.s, self.lw
        T, E = h.shape[0], s.experts
        # the router product in fp32; a shared expert's gate is one more row of the same matrix
        if s.router_bias:
            logits = torch.addmm(lw.router_b, h.float(), lw.router_w.t())
        else:
            logits = torch.mm(h.float(), lw.router_w.t())
        ids, wts = ops.moe_route(logits, lw.correction, s.top, s.groups, s.keep, softmax=s.score == "softmax",
                                 group_max=s.group_score == "max", weight_scale=s.weight_scale, experts=s.outputs,
                                 chosen_softmax=s.score == "chosen_softmax")
        offsets, perm, inv = ops.moe_sort(ids, s.outputs)
        extra = {}
        if s.identity:
            extra.update(ids=ids, x=h, num_real=E)
        if shared is not None:
            extra.update(shared=shared.contiguous())
        elif s.shared_ff:
            gu = self.r.linear(h, lw.shared_gate_up_w)
            extra.update(shared=self.r.linear(self._act(gu, s.shared_limit, s.shared_ff), lw.shared_down_w))
            if s.shared_gated:
                extra.update(shared_gate=logits[:, s.outputs:])
        rows = T * s.top
        if rows >= self.GROUPED_MIN_ROWS and not torch.cuda.is_current_stream_capturing():
            # many rows: library GEMMs per expert.  The experts' row ranges come to the host (one wait); when
            # the loads are near even, every expert's rows are padded to the largest count and the two products
            # are one batched GEMM each; otherwise one GEMM per expert on its range of the sorted rows.
            off = offsets.tolist()
            cap = -(-max(off[e + 1] - off[e] for e in range(E)) // 16) * 16
            if 0 < E * cap <= 2 * off[E]:
                xp = ops.moe_gather_rows(h, perm, rows, s.top, offsets=offsets, pad_to=cap, experts=E)
                gu = torch.bmm(xp.view(E, cap, -1), lw.gate_up_w.transpose(1, 2)).view(E * cap, 2 * s.ff)
                y = torch.bmm(self._act(gu, s.limit, s.ff).view(E, cap, s.ff), lw.down_w.transpose(1, 2)).view(E * cap, -1)
                extra["ids"] = ids
                return ops.moe_combine(y, inv, wts, T, s.top, offsets=offsets, pad_to=cap, **extra)
            xs = ops.moe_gather_rows(h, perm, rows, s.top)
            gu = torch.empty(rows, 2 * s.ff, dtype=h.dtype, device=h.device)
            for e in range(E):
                if off[e + 1] > off[e]:
                    torch.mm(xs[off[e]: off[e + 1]], lw.gate_up_w[e].t(), out=gu[off[e]: off[e + 1]])
            act = ops.moe_silu_and_mul(gu, s.limit)
            y = torch.empty(rows, h.shape[1], dtype=h.dtype, device=h.device)
            for e in range(E):
                if off[e + 1] > off[e]:
                    torch.mm(act[off[e]: off[e + 1]], lw.down_w[e].t(), out=y[off[e]: off[e + 1]])
        else:
            y = ops.moe_down_rows(ops.moe_gate_up_rows(h, lw.gate_up_w, offsets, perm, s.top, limit=s.limit), lw.down_w,
                                  offsets)
        return ops.moe_combine(y, inv, wts, T, s.top, **extra)


class HybridRunner(ModelRunner):
    def __init__(self, cfg: ModelConfig, weights: ModelWeights, dtype: torch.dtype, device, num_blocks: int,
                 max_num_seqs: int, max_model_len: int, tp_rank: int = 0, tp_size: int = 1, tp_group=None,
                 use_graphs: bool = True, decode_splits: Optional[int] = None, tiled_linears: Optional[bool] = None,
                 weight_fp8: bool = False, num_state_slots: Optional[int] = None):
        if cfg.family != "hybrid" or cfg.hybrid is None:
            raise ValueError("HybridRunner runs hybrid decoders")
        if tp_size != 1:
            raise ValueError("hybrid decoders run on one GPU (tensor_parallel_size 1)")
        if weight_fp8:
            raise ValueError("--quantization fp8 is not available for hybrid decoders")
        if dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise ValueError(f"dtype {dtype} not supported")
        self.cfg, self.w, self.dtype, self.device = cfg, weights, dtype, torch.device(device)
        self.spec = spec = cfg.hybrid
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.H, self.V, self.Vl = cfg.hidden_size, cfg.vocab_size, cfg.vocab_size
        self.vocab_sharded, self.vocab_offset = False, 0
        self.eps = cfg.rms_norm_eps
        self.L = len(spec.layers)
        self.num_blocks, self.max_num_seqs, self.max_model_len = int(num_blocks), int(max_num_seqs), int(max_model_len)
        self.max_blocks = (self.max_model_len + BLOCK_SIZE - 1) // BLOCK_SIZE
        self.use_graphs = use_graphs
        self.allow_eager_fallback = False
        self.capture_failures = self.tune_failures = 0
        self.oneshot = None
        self.oneshot_calls = self.fused_allreduce_norms = self.oneshot_key_reductions = self.oneshot_fallbacks = 0
        self._no_collectives = False
        self.decode_splits = decode_splits
        self.weight_fp8 = self.single_weight_copy = False
        self.tiled, self.tiled_policy, self._modes, self.tiled_shapes = None, "off", {}, {}
        # one spare slot past the engine's: padding rows of a decode graph park their state there
        self.num_state_slots = int(num_state_slots if num_state_slots is not None else max_num_seqs)
        dev = self.device
        self._rotary = {}
        # caches and state, one set per layer RUN (a looped layer: one per pass)
        self.runs = spec.runs()
        self.k_cache, self.v_cache, self.conv_state, self.rec_state, self.mixers = [], [], [], [], []
        self.latent_cache, self.ffs = [], []
        latent_of = {}                                  # layer index -> index of its latent pages
        for li, _ in self.runs if spec.arrangement == "sandwich" else ():
            L, lw = spec.layers[li], weights.layers[li]
            if L.kind == "general_delta":
                D = L.gdelta
                self.rec_state.append(torch.zeros(self.num_state_slots + 1, D.heads, D.dim, D.dim, dtype=torch.float32,
                                                  device=dev))
                self.mixers.append(GeneralDeltaMixer(D, lw, self, len(self.rec_state) - 1))
            else:
                A = L.lattn
                if A.kv_from is None:
                    # the latent pages, token-major with the rotated key part; where the matrix-core attention
                    # covers the sizes, the latent once more, channel-major
                    self.latent_cache.append((
                        torch.zeros(self.num_blocks, BLOCK_SIZE, A.kv_rank + A.rot_dim, dtype=dtype, device=dev),
                        torch.zeros(self.num_blocks, A.kv_rank, BLOCK_SIZE, dtype=dtype, device=dev)
                        if ops.latent_tiles_ok(dtype, A.kv_rank, A.rot_dim) else None))
                    latent_of[li] = len(self.latent_cache) - 1
                self.mixers.append(LatentAttention(A, lw, self, latent_of[li if A.kv_from is None else A.kv_from],
                                                   A.kv_from is None))
            self.ffs.append(MoEFeedForward(L.moe, lw, self) if L.moe is not None else None)
        pages_of = {}                                   # layer index -> index of its K/V pages
        for li, _ in self.runs if spec.arrangement == "parallel" else ():
            L, lw = spec.layers[li], weights.layers[li]
            A = L.battn
            if A.kv_from is None:
                self.k_cache.append(torch.zeros(self.num_blocks, A.kv_heads, BLOCK_SIZE, A.dim, dtype=dtype, device=dev))
                self.v_cache.append(torch.zeros(self.num_blocks, A.kv_heads, A.vdim, BLOCK_SIZE, dtype=dtype, device=dev))
                pages_of[li] = len(self.k_cache) - 1
            self.mixers.append(RotaryBlockAttention(A, lw, self, pages_of[li if A.kv_from is None else A.kv_from],
                                                    A.kv_from is None))
            self.ffs.append(MoEFeedForward(L.moe, lw, self) if L.moe is not None else None)
        for li, _ in self.runs if spec.arrangement == "pre" else ():
            L, lw = spec.layers[li], weights.layers[li]
            self.ffs.append(MoEFeedForward(L.moe, lw, self) if L.moe is not None else
                            ReluSquaredFF(lw, self) if L.ff and L.ff_act == "relu2" else None)
            if L.kind == "attention":
                A = L.battn
                self.k_cache.append(torch.zeros(self.num_blocks, A.kv_heads, BLOCK_SIZE, A.dim, dtype=dtype, device=dev))
                self.v_cache.append(torch.zeros(self.num_blocks, A.kv_heads, A.vdim, BLOCK_SIZE, dtype=dtype, device=dev))
                self.mixers.append(BlockAttention(A, lw, self, len(self.k_cache) - 1))
                continue
            if L.kind == "mingru":
                self.rec_state.append(torch.zeros(self.num_state_slots + 1, L.gru.width, dtype=torch.float32, device=dev))
                self.mixers.append(MinGRUMixer(L.gru, lw, self, len(self.rec_state) - 1))
                continue
            D = L.delta
            attn = None
            if L.attn is not None:
                A = L.attn
                self.k_cache.append(torch.zeros(self.num_blocks, A.kv_heads, BLOCK_SIZE, A.dim, dtype=dtype, device=dev))
                self.v_cache.append(torch.zeros(self.num_blocks, A.kv_heads, A.vdim, BLOCK_SIZE, dtype=dtype, device=dev))
                attn = WindowAttention(A, lw, self, len(self.k_cache) - 1)
            chans = 2 * D.kv_heads * D.dim + D.heads * D.vdim
            self.conv_state.append(torch.zeros(self.num_state_slots + 1, max(D.conv - 1, 0), chans, dtype=torch.float32,
                                               device=dev))
            self.rec_state.append(torch.zeros(self.num_state_slots + 1, D.heads, D.dim, D.vdim, dtype=torch.float32,
                                              device=dev))
            self.mixers.append((attn, DeltaMixer(D, lw, self, len(self.rec_state) - 1)))
        # the previous token of every live sequence (hashed previous-token embedding), beside the other state
        self.prev_tokens = torch.zeros(self.num_state_slots + 1, dtype=torch.int32, device=dev) \
            if spec.bigram is not None else None
        self._pos_freq = None
        if spec.sinusoid_base > 0:
            half = (self.H + 1) // 2
            f = float(spec.sinusoid_base) ** (-2.0 * np.arange(half, dtype=np.float64) / self.H)
            self._pos_freq = torch.from_numpy(f.astype(np.float32)).to(dev)
        B = self.max_num_seqs
        self._init_step_inputs(extra_i32=1)
        self.row_extra.fill_(self.num_state_slots)
        # the samplers want 16-byte aligned logit rows: the head is padded with zero rows to a multiple
        # of 8 and the logits are the first V columns of what it yields
        self.Vp = -(-self.V // 8) * 8
        self._forward = {"sandwich": self._forward_sandwich, "parallel": self._forward_parallel}.get(spec.arrangement,
                                                                                                     self._forward_pre)
        self.head_w = weights.lm_head
        if self.Vp != self.V:
            self.head_w = torch.zeros(self.Vp, self.H, dtype=dtype, device=dev)
            self.head_w[: self.V] = weights.lm_head
        self._init_tiled_copies(tiled_linears)
        self.logits_rows = torch.zeros(B, self.Vp, dtype=dtype, device=dev)
        self.logits = self.logits_rows[:, : self.V]
        self.graphs = {}
        self.buckets = batch_buckets(B)
        self._init_step_staging()
        # a decode step is B chunks of one row each
        self._dec_cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
        self._dec_seq = torch.arange(B, dtype=torch.int32, device=dev)
        # a decoded token is a tile of one row; its window's keys are spread over up to 8 workgroups
        self._dec_tiles = torch.stack([self._dec_seq, self._dec_seq, torch.ones_like(self._dec_seq)], dim=1).contiguous()
        widest = max([L.attn.heads * L.attn.vdim for L in spec.layers if L.attn is not None] + [0])
        self._attn_partial = torch.empty(max(self.MAX_KEY_SPLITS * B * widest, 4), dtype=torch.float32, device=dev)
        self.layer_trace = None                       # a list: _forward appends the residual after every layer run
        self._pair_tiles = {}                         # of the step at hand: heads -> device tiles
        self._dec_pairs = {}                          # of a decode step of max_num_seqs rows: heads -> device tiles

    # ------------------------------------------------------------------ #
    def rotary(self, rot_dims: int, base: float, scaling=None) -> torch.Tensor:
        key = (rot_dims, base, scaling)
        if key not in self._rotary:
            self._rotary[key] = rotary_table(rot_dims, base, self.max_blocks * BLOCK_SIZE, self.device, scaling)
        return self._rotary[key]

    def _decode_pair_tiles(self, heads: int) -> torch.Tensor:
        """Tiles of (row, head) pairs of a decode step: a row's tiles are adjacent, so the first b rows'
        tiles are a prefix."""
        if heads not in self._dec_pairs:
            cu = np.arange(self.max_num_seqs + 1, dtype=np.int64)
            self._dec_pairs[heads] = torch.from_numpy(ops.pair_tiles(cu, heads)).to(self.device)
        return self._dec_pairs[heads]

    def _chunk_pair_tiles(self, heads: int) -> torch.Tensor:
        if heads not in self._pair_tiles:
            self._pair_tiles[heads] = torch.from_numpy(ops.pair_tiles(self._step_cu, heads)).to(self.device, non_blocking=True)
        return self._pair_tiles[heads]

    MAX_KEY_SPLITS = 16

    def key_splits(self, b: StepBatch, a) -> dict:
        """Workgroups per tile for the window attention: more than one where one wave per (tile, block
        of heads) would leave most of the chip idle -- decoded tokens, and short or single prompts."""
        if b.tiles is None or self.dtype == torch.float32:
            return {}
        waves = int(b.tiles.shape[0]) * a.kv_heads * max((a.heads // a.kv_heads) // 4, 1)
        n = min(self.MAX_KEY_SPLITS, max(a.window // 64, 1), max(2048 // max(waves, 1), 1))
        if n <= 1:
            return {}
        need = n * b.num_tokens * a.heads * a.vdim
        if b.num_tokens <= self.max_num_seqs and need <= self._attn_partial.numel():
            return {"partial": self._attn_partial, "num_splits": n}      # static: a decode graph holds its address
        return {"partial": torch.empty(need, dtype=torch.float32, device=self.device), "num_splits": n}

    def block_key_splits(self, b: StepBatch, a) -> int:
        """Workgroups per tile for the block attention (as key_splits: decoded tokens and short prompts)."""
        if b.tiles is None or self.dtype == torch.float32:
            return 0
        rep = a.heads // a.kv_heads
        hb = 4 if rep % 4 == 0 else 3 if rep % 3 == 0 else 2 if rep % 2 == 0 else 1
        waves = int(b.tiles.shape[0]) * a.kv_heads * (rep // hb)
        span = a.block if a.block > 0 else self.max_model_len
        # about a wave per SIMD: every further split costs its fp32 partial sums and their merge (measured: a
        # 2048-token prompt of 16 heads 203 / 117 / 130 / 161 us with 1 / 2 / 4 / 8 splits, 32 decoded rows
        # 148 / 83 / 51 / 36 / 43 us with 1 / 2 / 4 / 8 / 16)
        n = min(self.MAX_KEY_SPLITS, max(span // 64, 1), max(1024 // max(waves, 1), 1))
        return n if n > 1 else 0

    def kv_cache_bytes_per_block(self) -> int:
        pages = self.k_cache + self.v_cache + [t for pair in self.latent_cache for t in pair if t is not None]
        return sum(t[0].numel() * t.element_size() for t in pages)

    def state_bytes_per_slot(self) -> int:
        return sum(t[0].numel() * t.element_size() for t in self.conv_state + self.rec_state) \
            + (4 if self.prev_tokens is not None else 0)

    def _init_tiled_copies(self, want: Optional[bool]) -> None:
        """Fragment-tiled second copies of the wide matrices for the weight-streaming GEMM of decode-sized
        steps (ModelRunner keeps the same kind of copy for its projections).  MI355_TILED_LINEARS=0 or
        tiled_linears=False: none (the row-major stream, mi355_linear_decode, serves those steps)."""
        import os
        self._tiled_w = {}
        if want is False or os.environ.get("MI355_TILED_LINEARS") == "0" or self.dtype == torch.float32:
            return
        mats = [self.head_w]
        for lw in self.w.layers:
            mats += [getattr(lw, n, None) for n in ("in_w", "delta_o_w", "attn_o_w", "gate_up_w", "down_w", "a2_w", "g2_w",
                                                    "o_w", "uq_w", "w2_w", "rg2_w", "up_w", "shared_gate_up_w", "shared_down_w",
                                                    "out_w")]
        for w in mats:
            # the kernel stages x in 512-wide K slices; narrow outputs leave too few workgroups to pay
            if w is not None and w.dim() == 2 and w.shape[1] % 512 == 0 and w.shape[0] >= 256 and w.shape[0] % 8 == 0:
                self._tiled_w[w.data_ptr()] = ops.tile_weights(w)

    def linear(self, x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
               bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x @ w.T (+ bias, in the accumulator's float32 ahead of the rounding).  Decode-sized row counts stream the weights once: through the fragment-tiled copy
        (K split over workgroups into fp32 slabs where one pass would leave most of the chip idle, a
        second launch adds the slabs) or, for matrices that have none, row-major through
        mi355_linear_decode.  A library GEMM otherwise (prefill; float32; odd widths)."""
        M, K = x.shape
        N = w.shape[0]
        ok16 = x.dtype != torch.float32 and x.stride(1) == 1 and (M == 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0
        tw = self._tiled_w.get(w.data_ptr()) if ok16 and M <= ops.LINEAR_DECODE_MAX_M else None
        if tw is not None:
            plan = ops.plan_linear_tiled(N, K, True, M)
            if plan is not None:
                tiles, groups = plan
                if out is None:
                    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
                if groups == 1:
                    return ops.linear_tiled(x, tw, N, bias=bias, out=out, tiles_per_wg=tiles)
                part = ops.linear_tiled(x, tw, N, tiles_per_wg=tiles, k_groups=groups, epilogue=ops.EPI_PARTIAL)
                return ops.sum_slabs(part, groups, out, bias=bias)
        if ok16 and M <= ops.LINEAR_DECODE_MAX_M and K % 32 == 0 and N % 4 == 0:
            return ops.linear_decode(x, w, bias, out=out)
        if bias is not None:
            return torch.addmm(bias, x, w.t()) if out is None else torch.addmm(bias, x, w.t(), out=out)
        if out is None:
            return torch.mm(x, w.t())
        return torch.mm(x, w.t(), out=out)

    def tune(self, bucket: int) -> dict:
        self._modes.setdefault(bucket, {})
        return self._modes[bucket]

    def warm_up(self) -> None:
        return None

    def capture(self, bucket: int) -> None:
        """As ModelRunner.capture; the warm-up and capture runs park every row's state in the spare
        slot, so that they cannot touch the state of live sequences."""
        if bucket in self.graphs:
            return
        saved = self.row_extra.clone()
        self.row_extra.fill_(self.num_state_slots)
        try:
            super().capture(bucket)
        finally:
            self.row_extra.copy_(saved)

    def _use_tiled(self, b: int) -> bool:
        return False

    # ------------------------------------------------------------------ #
    def _forward_sandwich(self, b: StepBatch) -> torch.Tensor:
        """All layers of the sandwich arrangement over one packed batch; returns the float32 residual
        stream [tokens, width]."""
        w, spec = self.w, self.spec
        G, eps, mult = spec.norm_groups, self.eps, spec.residual_mult
        resid = ops.embed_scale_f32(w.embed, b.ids, 1.0)
        ops.group_rms_norm_f32(resid, w.embed_norm, G, eps, out=resid)
        for ri, (li, _) in enumerate(self.runs):
            lw = w.layers[li]
            proj = self.linear(ops.group_rms_norm_f32(resid, lw.norm1, G, eps, dtype=self.dtype), lw.in_w)
            y = self.mixers[ri](proj, b)
            gate = proj[:, lw.seg["rg"][0]: lw.seg["rg"][0] + lw.seg["rg"][1]]
            ops.gated_norm_resid_f32(resid, y, gate, lw.rg1_b, lw.norm1b, G, eps, mult)
            if self.ffs[ri] is not None:
                h = ops.group_rms_norm_f32(resid, lw.norm2, G, eps, dtype=self.dtype)
                ops.gated_norm_resid_f32(resid, self.ffs[ri](h), self.linear(h, lw.rg2_w), lw.rg2_b, lw.norm2b, G, eps, mult)
            if self.layer_trace is not None:
                self.layer_trace.append(resid.clone())
        return resid

    def _forward_pre(self, b: StepBatch) -> torch.Tensor:
        """All layers over one packed batch; returns the float32 residual stream [tokens, width]."""
        w, spec = self.w, self.spec
        if spec.bigram is not None or self._pos_freq is not None:
            bg = spec.bigram
            resid = ops.embed_bigram_pos_f32(w.embed, b.ids, b.positions, w.bigram,
                                             (bg.buckets, bg.mul_prev, bg.mul_cur) if bg else None, b.cu_seqlens, b.tok_seq,
                                             b.state_slots, self.prev_tokens, self._pos_freq)
            if bg is not None:
                ops.prev_token_update(self.prev_tokens, b.ids, b.cu_seqlens, b.state_slots)
        else:
            resid = ops.embed_scale_f32(w.embed, b.ids, spec.embed_scale)
        x0 = resid.clone() if spec.loop_times > 1 else None
        pending = None                                 # a sub-layer output not yet added to the residual
        last = len(self.runs) - 1
        for ri, (li, t) in enumerate(self.runs):
            L, lw = spec.layers[li], w.layers[li]
            if t is not None and li == spec.loop_start:    # a pass begins: + embedding output (not the first) + its step vector
                ops.resid_add_f32(resid, other=x0 if t > 0 else None, rows=pending, vec=w.loop_step[t])
                pending = None
            h = ops.add_rms_norm_f32(resid, lw.norm1, self.eps, add=pending)    # the add rides in the norm's launch
            pending = None
            proj = self.linear(h, lw.in_w)
            mixer, ff = self.mixers[ri], self.ffs[ri]
            if not isinstance(mixer, tuple):
                pending = mixer(proj, b)
            elif mixer[0] is not None:
                attn, delta = mixer
                ops.rms_norm_mix_f32(resid, attn(proj, b), lw.attn_out_norm, delta(proj, b), lw.delta_out_norm,
                                     self.eps, 0.5)
            else:
                pending = mixer[1](proj, b)
            if ff is not None:
                pending = ff(ops.add_rms_norm_f32(resid, lw.norm2, self.eps, add=pending))
            elif L.ff:
                h = ops.add_rms_norm_f32(resid, lw.norm2, self.eps, add=pending)
                pending = self.linear(ops.gelu_tanh_and_mul(self.linear(h, lw.gate_up_w)), lw.down_w)
            if pending is not None and (ri == last or self.layer_trace is not None):
                ops.resid_add_f32(resid, rows=pending)
                pending = None
            if self.layer_trace is not None:
                self.layer_trace.append(resid.clone())
        return resid

    def _forward_parallel(self, b: StepBatch) -> torch.Tensor:
        """All layers of the parallel arrangement over one packed batch; returns the float32 residual
        stream [tokens, width].  Per layer: one norm (the previous layer's output rides in its launch),
        one product for everything that reads it, the attention and the gated activation writing side by
        side into one row, one product back: the sum of both sub-layers."""
        w, spec = self.w, self.spec
        if spec.learned_positions:
            resid = ops.embed_scale_pos_f32(w.embed, b.ids, spec.embed_scale, w.pos_embed, b.positions)
        else:
            resid = ops.embed_scale_f32(w.embed, b.ids, spec.embed_scale)
        T, pending, last = b.num_tokens, None, len(self.runs) - 1
        for ri, (li, _) in enumerate(self.runs):
            L, lw = spec.layers[li], w.layers[li]
            A = L.battn
            h = ops.add_rms_norm_f32(resid, lw.norm1, self.eps, add=pending)
            proj = self.linear(h, lw.in_w, bias=lw.in_b)
            n_attn = A.heads * A.vdim
            at, K = -(-n_attn // 8) * 8, lw.out_w.shape[1]          # the hidden units start on a 16-byte boundary
            row = (torch.zeros if at != n_attn else torch.empty)(T, K, dtype=self.dtype, device=self.device)
            self.mixers[ri](proj, b, row[:, :n_attn])
            if K > at:
                seg = lw.seg
                ops.gated_act_rows(proj[:, seg["gate"][0]: seg["gate"][0] + seg["gate"][1]],
                                   proj[:, seg["up"][0]: seg["up"][0] + seg["up"][1]],
                                   L.ff_limit if L.ff else L.moe.shared_limit, out=row[:, at:])
            pending = self.linear(row, lw.out_w)
            if self.ffs[ri] is not None:
                pending = self.ffs[ri](h, shared=pending)
            if ri == last or self.layer_trace is not None:
                ops.resid_add_f32(resid, rows=pending)
                pending = None
            if self.layer_trace is not None:
                self.layer_trace.append(resid.clone())
        return resid

    def _logits(self, resid: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Final norm, head and soft cap over the given residual rows."""
        if self.spec.arrangement == "sandwich":
            h = ops.group_rms_norm_f32(resid, self.w.final_norm, self.spec.norm_groups, self.eps, dtype=self.dtype)
        else:
            h = ops.add_rms_norm_f32(resid, self.w.final_norm, self.eps)
        z = self.linear(h, self.head_w, out=out)
        if self.spec.logit_softcap:
            ops.softcap(z, self.spec.logit_softcap)
        if self.spec.logit_scale != 1.0:
            z.mul_(self.spec.logit_scale)
        return z[:, : self.V]

    # ------------------------------------------------------------------ #
    def _decode_body(self, b: int) -> None:
        batch = StepBatch(self.ids[:b], self.positions[:b], self.slots[:b], self.block_tables[:b],
                          self._dec_cu[:b + 1], self._dec_seq[:b], self.row_extra[:b], self._dec_tiles[:b],
                          pair_tiles=lambda heads: self._decode_pair_tiles(heads)[: b * (-(-heads // 16))])
        resid = self._forward(batch)
        self._logits(resid, out=self.logits_rows[:b])
        self.greedy(self.logits[:b], self.next_ids[:b], ids_out=self.ids[:b])

    def run_prefill(self, token_ids, positions, slot_mapping, block_tables, cu_seqlens, context_lens, max_q_len: int,
                    sampling: Optional[dict] = None, logprobs: int = -1, prompt_logprobs=None, state_slots=None,
                    logit_rows=None):
        """As ModelRunner.run_prefill, over chunks that may be whole prompts, portions or single
        tokens.  `state_slots`: the state slot of every chunk.  `logit_rows` (packed row numbers):
        return float32 logits [rows, vocab] of those rows instead of sampling."""
        if state_slots is None:
            raise ValueError("hybrid decoders need the state slot of every chunk")
        self._step_state_slots = np.asarray(state_slots, dtype=np.int32)
        # rows go to the matrix cores in tiles of up to 16 rows of one chunk
        self._step_tiles = ops.query_tiles(cu_seqlens)
        self._step_cu, self._pair_tiles = np.asarray(cu_seqlens, dtype=np.int64), {}
        self._step_long = int(max_q_len) > 1
        if logit_rows is None:
            return super().run_prefill(token_ids, positions, slot_mapping, block_tables, cu_seqlens, context_lens,
                                       max_q_len, sampling=sampling, logprobs=logprobs, prompt_logprobs=prompt_logprobs)
        dev = self.device
        t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dev, dtype=dt, non_blocking=True)  # noqa: E731
        resid = self._run_chunks(t(token_ids, torch.int64), t(positions, torch.int64), t(slot_mapping, torch.int64),
                                 t(block_tables, torch.int32), t(cu_seqlens, torch.int32), t(context_lens, torch.int32),
                                 max_q_len)
        rows = np.asarray(logit_rows, dtype=np.int64)
        if rows.size == 0:
            torch.cuda.current_stream().synchronize()
            return np.zeros((0, self.V), dtype=np.float32)
        z = self._logits(resid.index_select(0, t(rows, torch.int64)))
        return z.float().cpu().numpy()

    def _run_chunks(self, token_ids, positions, slot_mapping, block_tables, cu_seqlens, context_lens=None,
                    max_q_len: int = 0) -> torch.Tensor:
        S = cu_seqlens.numel() - 1
        lens = (cu_seqlens[1:] - cu_seqlens[:-1]).to(torch.int64)
        tok_seq = torch.repeat_interleave(torch.arange(S, dtype=torch.int32, device=self.device), lens,
                                          output_size=int(token_ids.numel()))
        slots = torch.from_numpy(self._step_state_slots).to(self.device, non_blocking=True)
        tiles = torch.from_numpy(self._step_tiles).to(self.device, non_blocking=True)
        return self._forward(StepBatch(token_ids, positions, slot_mapping, block_tables.contiguous(), cu_seqlens,
                                       tok_seq, slots, tiles, self._step_long, pair_tiles=self._chunk_pair_tiles,
                                       context_lens=None if context_lens is None else context_lens.to(torch.int32).contiguous(),
                                       max_q_len=max_q_len))

    def prefill(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor,
                block_tables: torch.Tensor, cu_seqlens: torch.Tensor, context_lens: torch.Tensor,
                max_q_len: int, want_logits: bool = True, score=None):
        """As ModelRunner.prefill: packed prompts (or prompt chunks), eager."""
        resid = self._run_chunks(token_ids, positions, slot_mapping, block_tables, cu_seqlens, context_lens, max_q_len)
        if score is not None:
            k, srows, targets = score
            parts = []
            for a in range(0, srows.numel(), 1024):
                lg = self._logits(resid.index_select(0, srows[a:a + 1024]))
                parts.append(self._logprobs(lg, targets[a:a + 1024], k))
            self.prompt_scores = torch.cat(parts, dim=0)
        rows = (cu_seqlens[1:] - 1).to(torch.int64)
        logits = self._logits(resid.index_select(0, rows))
        nxt = torch.empty(logits.shape[0], dtype=torch.int64, device=self.device)
        self.greedy(logits, nxt)
        return nxt, (logits if want_logits else None)
