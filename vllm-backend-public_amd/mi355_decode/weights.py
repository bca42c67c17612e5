"""Model weights in the layout the kernels and GEMMs consume.

Per layer the q/k/v projections are concatenated into one [ (nh + 2*nkv) * d, H ]
matrix and gate/up into one [2F, H] matrix, all row-major [out, in] in the model
dtype.  Under tensor parallelism (one process per GPU) rank r keeps query heads
[r*nh/P, (r+1)*nh/P), the matching kv heads and the matching COLUMNS of o_proj
(row-parallel: partial sums are all-reduced).  With ``shard_mlp`` it also keeps
only rows [r*F/P, (r+1)*F/P) of gate_proj and up_proj and the matching columns of
down_proj (a second all-reduce per layer); otherwise the MLP is replicated.  With
``shard_vocab`` it keeps rows [r*V/P, (r+1)*V/P) of lm_head (greedy sampling then
max-reduces one key per sequence; full rows are gathered only for random sampling
and log-probabilities).  The embeddings are always replicated.

Sources: a local HF directory with *.safetensors (the harness serves models
from a local path, benchmark-mlflow/vllm_processor.py:29), an in-memory state
dict (tests), or seeded synthetic weights of the right shapes
(``--load-format dummy``; also the fallback when the directory holds no weight
files, because nothing can be downloaded).
"""
from __future__ import annotations

import glob
import json
import os
from dataclasses import dataclass, field
from typing import Callable, Optional

import torch

from .config import ModelConfig


@dataclass
class LayerWeights:
    qkv_w: torch.Tensor
    qkv_b: Optional[torch.Tensor]
    o_w: torch.Tensor
    gate_up_w: torch.Tensor
    down_w: torch.Tensor
    input_norm: torch.Tensor
    post_norm: torch.Tensor


@dataclass
class OPTLayerWeights:
    """One OPT decoder layer: q/k/v concatenated like LayerWeights; every projection has a bias,
    both norms a weight and a bias."""
    qkv_w: torch.Tensor
    qkv_b: torch.Tensor
    o_w: torch.Tensor
    o_b: torch.Tensor
    fc1_w: torch.Tensor
    fc1_b: torch.Tensor
    fc2_w: torch.Tensor
    fc2_b: torch.Tensor
    attn_norm_w: torch.Tensor
    attn_norm_b: torch.Tensor
    mlp_norm_w: torch.Tensor
    mlp_norm_b: torch.Tensor

    @property
    def down_w(self) -> torch.Tensor:          # [hidden, intermediate], the name the runner sizes its buffers by
        return self.fc2_w

    def tensors(self):
        return (self.qkv_w, self.qkv_b, self.o_w, self.o_b, self.fc1_w, self.fc1_b, self.fc2_w, self.fc2_b,
                self.attn_norm_w, self.attn_norm_b, self.mlp_norm_w, self.mlp_norm_b)


@dataclass
class HybridLayerWeights:
    """One layer of a hybrid decoder (config.HybridLayerSpec).  Everything that reads the layer's
    normed input is ONE matrix in_w [sum of segments, width]; `seg` maps a segment name to its
    (first column, width) in that projection's output:
      delta layer:     q | k | v | b | a | g
      parallel layer:  lq | lk | lv | lg (window attention and its per-head gate), then
                       q | k | v | b | a1 | g1 of the delta mixer (a1 / g1: the low-rank inputs of
                       decay and gate, widened by a2 / g2)
    q | k | v of the delta mixer are adjacent so that one convolution launch covers them (conv_w
    [q + k + v channels, taps]).  Per-head numbers and everything the recurrence reads besides the
    projections are float32."""
    norm1: torch.Tensor
    norm2: Optional[torch.Tensor]
    in_w: torch.Tensor
    seg: dict
    conv_w: torch.Tensor
    a_log: torch.Tensor                     # f32 [heads]
    dt_bias: torch.Tensor                   # f32 [heads] or [heads * dim]
    head_norm: torch.Tensor                 # f32 [vdim]
    delta_o_w: torch.Tensor
    a2_w: Optional[torch.Tensor] = None     # [heads * dim, rank]
    g2_w: Optional[torch.Tensor] = None     # [heads * vdim, rank]
    attn_temp: Optional[torch.Tensor] = None    # f32 [heads]
    attn_bias: Optional[torch.Tensor] = None    # f32 [heads]
    attn_o_w: Optional[torch.Tensor] = None
    attn_out_norm: Optional[torch.Tensor] = None
    delta_out_norm: Optional[torch.Tensor] = None
    gate_up_w: Optional[torch.Tensor] = None    # [2 ff, width]
    down_w: Optional[torch.Tensor] = None       # [width, ff]

    def tensors(self):
        return [t for t in vars(self).values() if isinstance(t, torch.Tensor)]


@dataclass
class SandwichLayerWeights:
    """One layer of a hybrid decoder in the "sandwich" arrangement (config.HybridSpec): a general
    delta rule or a latent attention, then a mixture of experts, each between a norm before and a
    gated, normed residual after.  Everything that reads the mixer's normed input is ONE matrix in_w
    (segments `seg`: name -> (first column, width) of the projection's output):
      general delta:     r | k | v | g | a | w1 | rg    (w1: the low-rank input of the decay, widened by w2_w)
      latent attention:  dq | dkv | g | rg              (dkv only if the layer makes its own latent)
    rg is the residual gate of the sub-layer.  Norm weights, biases, sinks, the router and its
    correction are float32; expert matrices are stacked [experts, ...]."""
    norm1: torch.Tensor                     # f32 [width] each
    norm1b: torch.Tensor
    in_w: torch.Tensor
    seg: dict
    rg1_b: torch.Tensor                     # f32 [width]
    o_w: torch.Tensor                       # [width, heads * dim] / [width, heads * vdim]
    # general delta rule
    w2_w: Optional[torch.Tensor] = None     # [heads * dim, rank]
    w0: Optional[torch.Tensor] = None       # f32 [heads * dim]
    a_b: Optional[torch.Tensor] = None      # f32 [heads * dim]
    head_norm: Optional[torch.Tensor] = None    # f32 [heads * dim]
    # latent attention
    dq_norm: Optional[torch.Tensor] = None  # f32 [q_rank]
    uq_w: Optional[torch.Tensor] = None     # [heads * (dim + rot_dim), q_rank]
    dkv_norm: Optional[torch.Tensor] = None     # f32 [kv_rank]
    uk_w: Optional[torch.Tensor] = None     # [heads, dim, kv_rank]
    uv_t: Optional[torch.Tensor] = None     # [heads, kv_rank, vdim]: the value up-projection, transposed per head
    sink: Optional[torch.Tensor] = None     # f32 [heads]
    # mixture of experts
    norm2: Optional[torch.Tensor] = None
    norm2b: Optional[torch.Tensor] = None
    rg2_w: Optional[torch.Tensor] = None    # [width, width]
    rg2_b: Optional[torch.Tensor] = None    # f32 [width]
    router_w: Optional[torch.Tensor] = None     # f32 [experts, width]
    correction: Optional[torch.Tensor] = None   # f32 [experts]
    gate_up_w: Optional[torch.Tensor] = None    # [experts, 2 ff, width]
    down_w: Optional[torch.Tensor] = None       # [experts, width, ff]

    def tensors(self):
        return [t for t in vars(self).values() if isinstance(t, torch.Tensor)]


@dataclass
class MixerLayerWeights:
    """One layer of a hybrid decoder in the "pre" arrangement whose mixer is a block attention or a
    per-channel gated recurrence (config.BlockAttnSpec / MinGRUSpec).  Everything that reads the
    mixer's normed input is ONE matrix in_w (segments `seg`: name -> (first column, width)):
      attention:  q | k | g        (g: the output gate, heads * vdim wide; the values are the keys)
      mingru:     z | x | g
    The feed-forward is dense (up_w, down_w), a mixture of experts (router_w float32 [experts +
    identity (+ 1), width]: the shared expert's gate row rides last in the fp32 router product;
    expert matrices stacked [experts, ...]; the shared expert as one more gate|up and down pair), or
    absent.  Norm weights are in the activation type, per-head numbers and biases float32."""
    norm1: torch.Tensor
    in_w: torch.Tensor
    seg: dict
    o_w: torch.Tensor
    q_norm: Optional[torch.Tensor] = None   # f32 [dim]
    k_norm: Optional[torch.Tensor] = None   # f32 [dim]
    r1: Optional[torch.Tensor] = None       # f32 [heads]
    r2: Optional[torch.Tensor] = None       # f32 [heads]
    z_b: Optional[torch.Tensor] = None      # f32 [width of the recurrence]
    x_b: Optional[torch.Tensor] = None
    norm2: Optional[torch.Tensor] = None
    up_w: Optional[torch.Tensor] = None     # dense: [ff, width]
    down_w: Optional[torch.Tensor] = None   # dense: [width, ff]; mixture: [experts, width, ff]
    router_w: Optional[torch.Tensor] = None
    correction: Optional[torch.Tensor] = None   # f32 [experts + identity]
    gate_up_w: Optional[torch.Tensor] = None    # [experts, 2 ff, width]
    shared_gate_up_w: Optional[torch.Tensor] = None     # [2 shared_ff, width]
    shared_down_w: Optional[torch.Tensor] = None        # [width, shared_ff]

    def tensors(self):
        return [t for t in vars(self).values() if isinstance(t, torch.Tensor)]


@dataclass
class ParallelLayerWeights:
    """One layer of a hybrid decoder in the "parallel" arrangement (one norm; the attention and the
    feed-forward both read it and their outputs are added).  Everything that reads the normed input
    in the activation type is ONE matrix in_w with one bias row in_b (zeros where a projection has
    none; None if no segment has one); segments `seg`: name -> (first column, width):
      q | [k | v] | g | [gate | up of the dense feed-forward or of the shared expert]
    (k and v are absent in a layer that attends to another layer's pages).  The two matrices that
    lead back to the residual are one as well, side by side along their inputs:
      out_w = [o | down]  [width, heads * vdim + ff]     (down: the dense or the shared expert's; absent: o alone)
    so that one product over the row [attention heads | activated hidden units] yields the sum of
    both sub-layers.  A mixture's router is float32 (router_w, router_b); its expert matrices are
    stacked."""
    norm1: torch.Tensor
    in_w: torch.Tensor
    in_b: Optional[torch.Tensor]
    seg: dict
    out_w: torch.Tensor
    sink: Optional[torch.Tensor] = None         # f32 [heads]: the score of the value-less term of the softmax denominator
    router_w: Optional[torch.Tensor] = None     # f32 [experts, width]
    router_b: Optional[torch.Tensor] = None     # f32 [experts]
    correction: Optional[torch.Tensor] = None   # f32 [experts], zeros: the choice is by the logits alone
    gate_up_w: Optional[torch.Tensor] = None    # [experts, 2 ff, width]
    down_w: Optional[torch.Tensor] = None       # [experts, width, ff]

    def tensors(self):
        return [t for t in vars(self).values() if isinstance(t, torch.Tensor)]


@dataclass
class ModelWeights:
    embed: torch.Tensor
    layers: list = field(default_factory=list)
    final_norm: torch.Tensor = None
    lm_head: torch.Tensor = None
    synthetic: bool = False
    pos_embed: Optional[torch.Tensor] = None     # learned positions (OPT): [max_positions + offset, hidden]
    final_norm_b: Optional[torch.Tensor] = None
    loop_step: Optional[torch.Tensor] = None     # hybrid decoders with a loop: [passes, width]
    embed_norm: Optional[torch.Tensor] = None    # hybrid decoders that norm the embedding: f32 [width]
    bigram: Optional[torch.Tensor] = None        # hashed previous-token embedding: [buckets + 1, width]

    def nbytes(self) -> int:
        total = self.embed.numel() * self.embed.element_size()
        if self.lm_head.untyped_storage().data_ptr() != self.embed.untyped_storage().data_ptr():
            total += self.lm_head.numel() * self.lm_head.element_size()
        total += self.final_norm.numel() * self.final_norm.element_size()
        for t in (self.pos_embed, self.final_norm_b, self.loop_step, self.embed_norm, self.bigram):
            if t is not None:
                total += t.numel() * t.element_size()
        for lw in self.layers:
            ts = lw.tensors() if isinstance(lw, (OPTLayerWeights, HybridLayerWeights, SandwichLayerWeights, MixerLayerWeights,
                                                 ParallelLayerWeights)) else \
                (lw.qkv_w, lw.qkv_b, lw.o_w, lw.gate_up_w, lw.down_w, lw.input_norm, lw.post_norm)
            for t in ts:
                if t is not None:
                    total += t.numel() * t.element_size()
        return total


def _shard_heads(cfg: ModelConfig, tp_rank: int, tp_size: int):
    nh, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    if nh % tp_size or nkv % tp_size:
        raise ValueError(f"tensor_parallel_size {tp_size} must divide num_attention_heads {nh} and "
                         f"num_key_value_heads {nkv}")
    nh_l, nkv_l = nh // tp_size, nkv // tp_size
    return nh_l, nkv_l, slice(tp_rank * nh_l * cfg.head_dim, (tp_rank + 1) * nh_l * cfg.head_dim), \
        slice(tp_rank * nkv_l * cfg.head_dim, (tp_rank + 1) * nkv_l * cfg.head_dim)


def _shard_mlp(cfg: ModelConfig, tp_rank: int, tp_size: int) -> slice:
    F = cfg.intermediate_size
    if F % tp_size:
        raise ValueError(f"tensor_parallel_size {tp_size} must divide intermediate_size {F}")
    return slice(tp_rank * (F // tp_size), (tp_rank + 1) * (F // tp_size))


def _shard_vocab(cfg: ModelConfig, tp_rank: int, tp_size: int) -> slice:
    V = cfg.vocab_size
    if V % (16 * tp_size):
        raise ValueError(f"16 * tensor_parallel_size {tp_size} must divide vocab_size {V} to shard lm_head")
    return slice(tp_rank * (V // tp_size), (tp_rank + 1) * (V // tp_size))


def from_getter(cfg: ModelConfig, get: Callable[[str], torch.Tensor], dtype: torch.dtype, device,
                tp_rank: int = 0, tp_size: int = 1, num_layers: Optional[int] = None,
                shard_mlp: bool = False, shard_vocab: bool = False) -> ModelWeights:
    """``get(name)`` returns the full (unsharded) CPU tensor of an HF parameter."""
    if cfg.family == "opt":
        return _opt_from_getter(cfg, get, dtype, device, tp_size, num_layers)
    if cfg.family == "hybrid":
        return _hybrid_from_getter(cfg, get, dtype, device, tp_size, num_layers)
    _, _, qs, ks = _shard_heads(cfg, tp_rank, tp_size)
    fs = _shard_mlp(cfg, tp_rank, tp_size) if shard_mlp else slice(None)

    def put(t: torch.Tensor) -> torch.Tensor:
        return t.to(dtype).contiguous().to(device)

    L = num_layers if num_layers is not None else cfg.num_hidden_layers
    w = ModelWeights(embed=put(get("model.embed_tokens.weight")))
    for i in range(L):
        p = f"model.layers.{i}."
        q, k, v = (get(p + f"self_attn.{n}_proj.weight") for n in "qkv")
        qkv_w = torch.cat([q[qs], k[ks], v[ks]], dim=0)
        qkv_b = None
        if cfg.attention_bias:
            qb, kb, vb = (get(p + f"self_attn.{n}_proj.bias") for n in "qkv")
            qkv_b = put(torch.cat([qb[qs], kb[ks], vb[ks]], dim=0))
        o = get(p + "self_attn.o_proj.weight")[:, qs]
        gu = torch.cat([get(p + "mlp.gate_proj.weight")[fs], get(p + "mlp.up_proj.weight")[fs]], dim=0)
        w.layers.append(LayerWeights(
            qkv_w=put(qkv_w), qkv_b=qkv_b, o_w=put(o), gate_up_w=put(gu),
            down_w=put(get(p + "mlp.down_proj.weight")[:, fs]),
            input_norm=put(get(p + "input_layernorm.weight")),
            post_norm=put(get(p + "post_attention_layernorm.weight"))))
    w.final_norm = put(get("model.norm.weight"))
    vs = _shard_vocab(cfg, tp_rank, tp_size) if shard_vocab else slice(None)
    w.lm_head = w.embed[vs] if cfg.tie_word_embeddings else put(get("lm_head.weight")[vs])
    return w


def _opt_only_one_gpu(tp_size: int) -> None:
    if tp_size != 1:
        raise ValueError("OPT models run on one GPU (tensor_parallel_size 1): the harness deploys them as its "
                         "single-process plumbing case")


def _opt_from_getter(cfg: ModelConfig, get, dtype, device, tp_size: int, num_layers: Optional[int]) -> ModelWeights:
    """HF OPT parameter names (model.decoder.*; transformers models/opt/modeling_opt.py).  Some
    published OPT checkpoints store the decoder without the `model.` prefix (`decoder.*`) next to a
    separate, tied `lm_head.weight`: both namings load, the lm_head copy is not read."""
    _opt_only_one_gpu(tp_size)
    get_as_named = get

    def get(name):                                       # noqa: F811  model.decoder.X, else decoder.X
        try:
            return get_as_named(name)
        except KeyError:
            if not name.startswith("model."):
                raise
            try:
                return get_as_named(name[len("model."):])
            except KeyError:
                raise KeyError(f"{name} (or {name[len('model.'):]}) not found in the checkpoint") from None

    def put(t: torch.Tensor) -> torch.Tensor:
        return t.to(dtype).contiguous().to(device)

    D = "model.decoder."
    L = num_layers if num_layers is not None else cfg.num_hidden_layers
    w = ModelWeights(embed=put(get(D + "embed_tokens.weight")), pos_embed=put(get(D + "embed_positions.weight")))
    for i in range(L):
        p = f"{D}layers.{i}."
        w.layers.append(OPTLayerWeights(
            qkv_w=put(torch.cat([get(p + f"self_attn.{n}_proj.weight") for n in "qkv"], dim=0)),
            qkv_b=put(torch.cat([get(p + f"self_attn.{n}_proj.bias") for n in "qkv"], dim=0)),
            o_w=put(get(p + "self_attn.out_proj.weight")), o_b=put(get(p + "self_attn.out_proj.bias")),
            fc1_w=put(get(p + "fc1.weight")), fc1_b=put(get(p + "fc1.bias")),
            fc2_w=put(get(p + "fc2.weight")), fc2_b=put(get(p + "fc2.bias")),
            attn_norm_w=put(get(p + "self_attn_layer_norm.weight")), attn_norm_b=put(get(p + "self_attn_layer_norm.bias")),
            mlp_norm_w=put(get(p + "final_layer_norm.weight")), mlp_norm_b=put(get(p + "final_layer_norm.bias"))))
    w.final_norm = put(get(D + "final_layer_norm.weight"))
    w.final_norm_b = put(get(D + "final_layer_norm.bias"))
    w.lm_head = w.embed                                  # tied (OPTForCausalLM ties lm_head to embed_tokens)
    return w


def _opt_synthetic(cfg: ModelConfig, dtype, device, seed: int, tp_size: int, num_layers: Optional[int],
                   std: float) -> ModelWeights:
    _opt_only_one_gpu(tp_size)
    H, F, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    gen = torch.Generator(device=device).manual_seed(seed)

    def mat(*shape):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, std, generator=gen)

    def ones():
        return torch.ones(H, dtype=dtype, device=device)

    L = num_layers if num_layers is not None else cfg.num_hidden_layers
    w = ModelWeights(embed=mat(V, H), synthetic=True,
                     pos_embed=mat(cfg.max_position_embeddings + cfg.position_offset, H))
    for _ in range(L):
        w.layers.append(OPTLayerWeights(
            qkv_w=mat(3 * H, H), qkv_b=mat(3 * H), o_w=mat(H, H), o_b=mat(H), fc1_w=mat(F, H), fc1_b=mat(F),
            fc2_w=mat(H, F), fc2_b=mat(H), attn_norm_w=ones(), attn_norm_b=mat(H), mlp_norm_w=ones(),
            mlp_norm_b=mat(H)))
    w.final_norm, w.final_norm_b = ones(), mat(H)
    w.lm_head = w.embed
    return w


def _hybrid_one_gpu(tp_size: int, num_layers) -> None:
    if tp_size != 1:
        raise ValueError("hybrid decoders run on one GPU (tensor_parallel_size 1)")
    if num_layers is not None:
        raise ValueError("hybrid decoders run all their layers (no layer override)")


def _hybrid_from_getter(cfg: ModelConfig, get, dtype, device, tp_size: int, num_layers) -> ModelWeights:
    """Lozupel checkpoints: 'embed', 'head', 'final.norm', 'loop.step', and per layer i 'l<i>.norm1',
    'l<i>.norm2', 'l<i>.mix.*' (a parallel layer's two mixers under '.left' / '.right'),
    'l<i>.mlp.gate|up|down'.  Linear weights are [out, in]."""
    _hybrid_one_gpu(tp_size, num_layers)
    spec = cfg.hybrid
    W = cfg.hidden_size
    if spec.arrangement == "sandwich":
        return _sandwich_from_getter(cfg, get, dtype, device)
    if cfg.architecture == "Tafisun":
        return _tafisun_from_getter(cfg, get, dtype, device)
    if spec.arrangement == "parallel":
        return _bemulorn_from_getter(cfg, get, dtype, device)

    def put(t, dt=dtype):
        return t.to(dt).contiguous().to(device)

    def f32(t):
        return put(t.reshape(-1), torch.float32)

    def fuse(parts):
        seg, at = {}, 0
        for name, t in parts:
            if t.dim() != 2 or t.shape[1] != W:
                raise ValueError(f"segment {name}: shape {tuple(t.shape)}, expected [*, {W}]")
            seg[name] = (at, int(t.shape[0]))
            at += -(-int(t.shape[0]) // 8) * 8          # every segment starts on a 16-byte boundary of the output row
        full = torch.zeros(at, W, dtype=parts[0][1].dtype)
        for name, t in parts:
            full[seg[name][0]: seg[name][0] + seg[name][1]] = t
        return put(full), seg

    def expect(name, t, shape):
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    w = ModelWeights(embed=put(expect("embed", get("embed"), (cfg.vocab_size, W))))
    for i, L in enumerate(spec.layers):
        p = f"l{i}."
        m = p + "mix." + ("right." if L.kind == "parallel" else "")
        D = L.delta
        qk, vv = D.kv_heads * D.dim, D.heads * D.vdim
        parts = []
        if L.kind == "parallel":
            A, a = L.attn, p + "mix.left."
            parts += [("lq", expect(a + "q", get(a + "q"), (A.heads * A.dim, W))),
                      ("lk", expect(a + "k", get(a + "k"), (A.kv_heads * A.dim, W))),
                      ("lv", expect(a + "v", get(a + "v"), (A.kv_heads * A.vdim, W))),
                      ("lg", expect(a + "g", get(a + "g"), (A.heads, W)))]
        parts += [("q", expect(m + "q", get(m + "q"), (qk, W))), ("k", expect(m + "k", get(m + "k"), (qk, W))),
                  ("v", expect(m + "v", get(m + "v"), (vv, W))), ("b", expect(m + "b", get(m + "b"), (D.heads, W)))]
        if D.per_channel:
            parts += [("a1", get(m + "a1")), ("g1", get(m + "g1"))]
        else:
            parts += [("a", expect(m + "a", get(m + "a"), (D.heads, W))), ("g", expect(m + "g", get(m + "g"), (vv, W)))]
        in_w, seg = fuse(parts)
        conv = torch.cat([expect(m + n + ".conv", get(m + n + ".conv"), (c, D.conv))
                          for n, c in (("q", qk), ("k", qk), ("v", vv))], dim=0)
        lw = HybridLayerWeights(
            norm1=put(get(p + "norm1").reshape(1)), norm2=put(get(p + "norm2").reshape(1)) if L.ff else None,
            in_w=in_w, seg=seg, conv_w=put(conv), a_log=f32(expect(m + "A_log", get(m + "A_log"), (D.heads,))),
            dt_bias=f32(expect(m + "dt_bias", get(m + "dt_bias"), (D.heads * D.dim if D.per_channel else D.heads,))),
            head_norm=f32(expect(m + "norm", get(m + "norm"), (D.vdim,))),
            delta_o_w=put(expect(m + "o", get(m + "o"), (W, vv))))
        if D.per_channel:
            lw.a2_w = put(expect(m + "a2", get(m + "a2"), (D.heads * D.dim, seg["a1"][1])))
            lw.g2_w = put(expect(m + "g2", get(m + "g2"), (vv, seg["g1"][1])))
        if L.kind == "parallel":
            A, a = L.attn, p + "mix.left."
            lw.attn_temp, lw.attn_bias = f32(expect(a + "temp", get(a + "temp"), (A.heads,))), \
                f32(expect(a + "pb", get(a + "pb"), (A.heads,)))
            lw.attn_o_w = put(expect(a + "o", get(a + "o"), (W, A.heads * A.vdim)))
            lw.attn_out_norm = put(expect(a + "out", get(a + "out"), (W,)))
            lw.delta_out_norm = put(expect(m + "out", get(m + "out"), (W,)))
        if L.ff:
            g, u = get(p + "mlp.gate"), get(p + "mlp.up")
            lw.gate_up_w = put(torch.cat([expect(p + "mlp.gate", g, (L.ff, W)), expect(p + "mlp.up", u, (L.ff, W))], dim=0))
            lw.down_w = put(expect(p + "mlp.down", get(p + "mlp.down"), (W, L.ff)))
        w.layers.append(lw)
    w.final_norm = put(get("final.norm").reshape(1))
    w.lm_head = put(expect("head", get("head"), (cfg.vocab_size, W)))
    if spec.loop_times > 0:
        w.loop_step = put(expect("loop.step", get("loop.step"), (spec.loop_times, W)))
    return w


def _fuse_segments(parts, W: int, put):
    """One matrix of all the projections that read the same input; every segment starts on a 16-byte
    boundary of the output row.  Returns (matrix, {name: (first column, width)})."""
    seg, at = {}, 0
    for name, t in parts:
        if t.dim() != 2 or t.shape[1] != W:
            raise ValueError(f"segment {name}: shape {tuple(t.shape)}, expected [*, {W}]")
        seg[name] = (at, int(t.shape[0]))
        at += -(-int(t.shape[0]) // 8) * 8
    full = torch.zeros(at, W, dtype=parts[0][1].dtype)
    for name, t in parts:
        full[seg[name][0]: seg[name][0] + seg[name][1]] = t
    return put(full), seg


def _sandwich_from_getter(cfg: ModelConfig, get, dtype, device) -> ModelWeights:
    """Tativik checkpoints: 'embed', 'embed.norm', 'final.norm', 'head', and per layer i 'l<i>.norm1|norm1b|
    norm2|norm2b', 'l<i>.rg1|rg2' with '.b', 'l<i>.mix.*' (general delta: r k v g a a.b w1 w2 w0 norm o;
    latent attention: dq dq.norm uq [dkv dkv.norm] uk uv sink g o), 'l<i>.mlp.router|correction' and
    'l<i>.mlp.e<j>.gate|up|down'.  Linear weights are [out, in]."""
    spec, W = cfg.hybrid, cfg.hidden_size

    def put(t, dt=dtype):
        return t.to(dt).contiguous().to(device)

    def f32(t):
        return put(t.reshape(-1), torch.float32)

    def expect(name, shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    w = ModelWeights(embed=put(expect("embed", (cfg.vocab_size, W))), embed_norm=f32(expect("embed.norm", (W,))))
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", f"l{i}.mix."
        kw = dict(norm1=f32(expect(p + "norm1", (W,))), norm1b=f32(expect(p + "norm1b", (W,))),
                  rg1_b=f32(expect(p + "rg1.b", (W,))))
        rg1 = ("rg", expect(p + "rg1", (W, W)))
        if L.kind == "general_delta":
            D = L.gdelta
            C = D.heads * D.dim
            w1 = get(m + "w1")
            in_w, seg = _fuse_segments([(n, expect(m + n, (C, W))) for n in "rkvga"] + [("w1", w1), rg1], W, put)
            kw.update(in_w=in_w, seg=seg, o_w=put(expect(m + "o", (W, C))), w2_w=put(expect(m + "w2", (C, w1.shape[0]))),
                      w0=f32(expect(m + "w0", (C,))), a_b=f32(expect(m + "a.b", (C,))),
                      head_norm=f32(expect(m + "norm", (C,))))
        else:
            A = L.lattn
            if A.q_rank <= 0:                             # not named by the configuration: the tensor's shape gives it
                A.q_rank = int(get(m + "dq").shape[0])
            parts = [("dq", expect(m + "dq", (A.q_rank, W)))]
            if A.kv_from is None:
                parts.append(("dkv", expect(m + "dkv", (A.kv_rank + A.rot_dim, W))))
                kw["dkv_norm"] = f32(expect(m + "dkv.norm", (A.kv_rank,)))
            in_w, seg = _fuse_segments(parts + [("g", expect(m + "g", (A.heads, W))), rg1], W, put)
            uv = expect(m + "uv", (A.heads * A.vdim, A.kv_rank)).view(A.heads, A.vdim, A.kv_rank)
            kw.update(in_w=in_w, seg=seg, o_w=put(expect(m + "o", (W, A.heads * A.vdim))),
                      dq_norm=f32(expect(m + "dq.norm", (A.q_rank,))),
                      uq_w=put(expect(m + "uq", (A.heads * (A.dim + A.rot_dim), A.q_rank))),
                      uk_w=put(expect(m + "uk", (A.heads * A.dim, A.kv_rank)).view(A.heads, A.dim, A.kv_rank)),
                      uv_t=put(uv.transpose(1, 2)), sink=f32(expect(m + "sink", (A.heads,))))
        if L.moe is not None:
            M, q = L.moe, p + "mlp."
            gu = torch.stack([torch.cat([expect(f"{q}e{e}.gate", (M.ff, W)), expect(f"{q}e{e}.up", (M.ff, W))], dim=0)
                              for e in range(M.experts)])
            kw.update(norm2=f32(expect(p + "norm2", (W,))), norm2b=f32(expect(p + "norm2b", (W,))),
                      rg2_w=put(expect(p + "rg2", (W, W))), rg2_b=f32(expect(p + "rg2.b", (W,))),
                      router_w=put(expect(q + "router", (M.experts, W)), torch.float32),
                      correction=f32(expect(q + "correction", (M.experts,))), gate_up_w=put(gu),
                      down_w=put(torch.stack([expect(f"{q}e{e}.down", (W, M.ff)) for e in range(M.experts)])))
        w.layers.append(SandwichLayerWeights(**kw))
    w.final_norm = f32(expect("final.norm", (W,)))
    w.lm_head = put(expect("head", (cfg.vocab_size, W)))
    return w


def _tafisun_from_getter(cfg: ModelConfig, get, dtype, device) -> ModelWeights:
    """Tafisun checkpoints: 'embed', 'bigram', 'final.norm', 'head', and per layer i 'l<i>.norm1|norm2',
    'l<i>.mix.*' (attention: q k q.norm k.norm r1 r2 g o; mingru: z z.b x x.b g o), 'l<i>.mlp.up|down'
    (dense) or 'l<i>.mlp.router|correction', 'l<i>.mlp.e<j>.gate|up|down' and
    'l<i>.mlp.shared.gate|up|down|sg' (mixture).  Linear weights are [out, in]."""
    spec, W = cfg.hybrid, cfg.hidden_size

    def put(t, dt=dtype):
        return t.to(dt).contiguous().to(device)

    def f32(t):
        return put(t.reshape(-1), torch.float32)

    def expect(name, shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    w = ModelWeights(embed=put(expect("embed", (cfg.vocab_size, W))))
    if spec.bigram is not None:
        w.bigram = put(expect("bigram", (spec.bigram.buckets + 1, W)))
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", f"l{i}.mix."
        if L.kind == "attention":
            A = L.battn
            in_w, seg = _fuse_segments([("q", expect(m + "q", (A.heads * A.dim, W))), ("k", expect(m + "k", (A.kv_heads * A.dim, W))),
                                        ("g", expect(m + "g", (A.heads * A.vdim, W)))], W, put)
            lw = MixerLayerWeights(norm1=put(expect(p + "norm1", (W,))), in_w=in_w, seg=seg,
                                   o_w=put(expect(m + "o", (W, A.heads * A.vdim))),
                                   q_norm=f32(expect(m + "q.norm", (A.dim,))), k_norm=f32(expect(m + "k.norm", (A.dim,))),
                                   r1=f32(expect(m + "r1", (A.heads,))), r2=f32(expect(m + "r2", (A.heads,))))
        else:
            C = L.gru.width
            in_w, seg = _fuse_segments([(n, expect(m + n, (C, W))) for n in "zxg"], W, put)
            lw = MixerLayerWeights(norm1=put(expect(p + "norm1", (W,))), in_w=in_w, seg=seg, o_w=put(expect(m + "o", (W, C))),
                                   z_b=f32(expect(m + "z.b", (C,))), x_b=f32(expect(m + "x.b", (C,))))
        q = p + "mlp."
        if L.ff:
            lw.norm2 = put(expect(p + "norm2", (W,)))
            lw.up_w, lw.down_w = put(expect(q + "up", (L.ff, W))), put(expect(q + "down", (W, L.ff)))
        elif L.moe is not None:
            M = L.moe
            lw.norm2 = put(expect(p + "norm2", (W,)))
            router = [expect(q + "router", (M.outputs, W))]
            if M.shared_ff:
                router.append(expect(q + "shared.sg", (1, W)))
                lw.shared_gate_up_w = put(torch.cat([expect(q + "shared.gate", (M.shared_ff, W)),
                                                     expect(q + "shared.up", (M.shared_ff, W))], dim=0))
                lw.shared_down_w = put(expect(q + "shared.down", (W, M.shared_ff)))
            lw.router_w = put(torch.cat(router, dim=0), torch.float32)
            lw.correction = f32(expect(q + "correction", (M.outputs,)))
            lw.gate_up_w = put(torch.stack([torch.cat([expect(f"{q}e{e}.gate", (M.ff, W)), expect(f"{q}e{e}.up", (M.ff, W))],
                                                      dim=0) for e in range(M.experts)]))
            lw.down_w = put(torch.stack([expect(f"{q}e{e}.down", (W, M.ff)) for e in range(M.experts)]))
        w.layers.append(lw)
    w.final_norm = put(expect("final.norm", (W,)))
    w.lm_head = put(expect("head", (cfg.vocab_size, W)))
    return w


def _bemulorn_from_getter(cfg: ModelConfig, get, dtype, device) -> ModelWeights:
    """Bemulorn checkpoints: 'embed', 'pos', 'final.norm', 'head', and per layer i 'l<i>.norm1',
    'l<i>.mix.q|k|v' with '.b', 'l<i>.mix.g|o' (no k, v in a layer that reads another layer's pages),
    'l<i>.mlp.gate|up|down' (dense) or 'l<i>.mlp.router' with '.b', 'l<i>.mlp.e<j>.gate|up|down' and
    'l<i>.mlp.shared.gate|up|down' (mixture).  Linear weights are [out, in]."""
    spec, W = cfg.hybrid, cfg.hidden_size

    def put(t, dt=dtype):
        return t.to(dt).contiguous().to(device)

    def f32(t):
        return put(t.reshape(-1), torch.float32)

    def expect(name, shape):
        t = get(name)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    w = ModelWeights(embed=put(expect("embed", (cfg.vocab_size, W))))
    pos = get("pos")
    if pos.dim() != 2 or pos.shape[1] != W:
        raise ValueError(f"pos: shape {tuple(pos.shape)}, expected [positions, {W}]")
    w.pos_embed = put(pos)
    for i, L in enumerate(spec.layers):
        p, m, q = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        A = L.battn
        parts = [("q", expect(m + "q", (A.heads * A.dim, W)))]
        if A.kv_from is None:
            parts += [("k", expect(m + "k", (A.kv_heads * A.dim, W))), ("v", expect(m + "v", (A.kv_heads * A.vdim, W)))]
        parts.append(("g", expect(m + "g", (A.heads, W))))
        outs = [expect(m + "o", (W, A.heads * A.vdim))]
        ff = L.ff if L.ff else (L.moe.shared_ff if L.moe is not None else 0)
        if ff:
            r = q if L.ff else q + "shared."
            parts += [("gate", expect(r + "gate", (ff, W))), ("up", expect(r + "up", (ff, W)))]
            outs.append(expect(r + "down", (W, ff)))
        in_w, seg = _fuse_segments(parts, W, put)
        in_b = None
        if A.bias:
            b = torch.zeros(in_w.shape[0], dtype=torch.float32)
            for n, _ in parts[: 3 if A.kv_from is None else 1]:
                b[seg[n][0]: seg[n][0] + seg[n][1]] = expect(m + n + ".b", (seg[n][1],)).float()
            in_b = put(b)
        # the row that out_w multiplies: the heads, then the activated hidden units on a 16-byte boundary
        n_attn = -(-A.heads * A.vdim // 8) * 8
        out_w = torch.zeros(W, n_attn + ff, dtype=outs[0].dtype)
        out_w[:, : A.heads * A.vdim] = outs[0]
        if ff:
            out_w[:, n_attn:] = outs[1]
        lw = ParallelLayerWeights(norm1=put(expect(p + "norm1", (W,))), in_w=in_w, in_b=in_b, seg=seg, out_w=put(out_w),
                                  sink=torch.full((A.heads,), float(A.sink), dtype=torch.float32, device=device)
                                  if A.sink is not None else None)
        if L.moe is not None:
            M = L.moe
            lw.router_w = put(expect(q + "router", (M.experts, W)), torch.float32)
            lw.router_b = f32(expect(q + "router.b", (M.experts,))) if M.router_bias else None
            lw.correction = torch.zeros(M.experts, dtype=torch.float32, device=device)
            lw.gate_up_w = put(torch.stack([torch.cat([expect(f"{q}e{e}.gate", (M.ff, W)), expect(f"{q}e{e}.up", (M.ff, W))],
                                                      dim=0) for e in range(M.experts)]))
            lw.down_w = put(torch.stack([expect(f"{q}e{e}.down", (W, M.ff)) for e in range(M.experts)]))
        w.layers.append(lw)
    w.final_norm = put(expect("final.norm", (W,)))
    w.lm_head = put(expect("head", (cfg.vocab_size, W)))
    return w


def bemulorn_synthetic_state(cfg: ModelConfig, seed: int = 0, device="cpu", dtype=torch.float32) -> dict:
    """Seeded random tensors under a Bemulorn checkpoint's names (benchmarks and tests: nothing can be
    downloaded)."""
    spec, W = cfg.hybrid, cfg.hidden_size
    gen = torch.Generator(device=device).manual_seed(seed)

    def mat(*shape, s=1.0):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, s, generator=gen)

    def near(value, *shape, s=0.1):
        return torch.full(shape, float(value), dtype=dtype, device=device) + mat(*shape, s=s)

    st = {"embed": mat(cfg.vocab_size, W), "pos": mat(cfg.max_position_embeddings, W, s=0.5),
          "head": mat(cfg.vocab_size, W, s=W ** -0.5), "final.norm": near(1.0, W)}
    for i, L in enumerate(spec.layers):
        p, m, q = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        A = L.battn
        st[p + "norm1"] = near(1.0, W)
        st[m + "q"], st[m + "q.b"] = mat(A.heads * A.dim, W, s=W ** -0.5), mat(A.heads * A.dim, s=0.2)
        if A.kv_from is None:
            st[m + "k"], st[m + "k.b"] = mat(A.kv_heads * A.dim, W, s=W ** -0.5), mat(A.kv_heads * A.dim, s=0.2)
            st[m + "v"], st[m + "v.b"] = mat(A.kv_heads * A.vdim, W, s=W ** -0.5), mat(A.kv_heads * A.vdim, s=0.2)
        st[m + "g"] = mat(A.heads, W, s=W ** -0.5)
        st[m + "o"] = mat(W, A.heads * A.vdim, s=(A.heads * A.vdim) ** -0.5)
        if L.ff:
            st[q + "gate"], st[q + "up"] = mat(L.ff, W, s=W ** -0.5), mat(L.ff, W, s=W ** -0.5)
            st[q + "down"] = mat(W, L.ff, s=L.ff ** -0.5)
        elif L.moe is not None:
            M = L.moe
            st[q + "router"], st[q + "router.b"] = mat(M.experts, W, s=W ** -0.5), mat(M.experts, s=0.3)
            for e in range(M.experts):
                st[f"{q}e{e}.gate"], st[f"{q}e{e}.up"] = mat(M.ff, W, s=W ** -0.5), mat(M.ff, W, s=W ** -0.5)
                st[f"{q}e{e}.down"] = mat(W, M.ff, s=M.ff ** -0.5)
            if M.shared_ff:
                st[q + "shared.gate"], st[q + "shared.up"] = mat(M.shared_ff, W, s=W ** -0.5), mat(M.shared_ff, W, s=W ** -0.5)
                st[q + "shared.down"] = mat(W, M.shared_ff, s=M.shared_ff ** -0.5)
    return st


def tafisun_synthetic_state(cfg: ModelConfig, seed: int = 0, device="cpu", dtype=torch.float32) -> dict:
    """Seeded random tensors under a Tafisun checkpoint's names (benchmarks and tests: nothing can be
    downloaded)."""
    spec, W = cfg.hybrid, cfg.hidden_size
    gen = torch.Generator(device=device).manual_seed(seed)

    def mat(*shape, s=1.0):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, s, generator=gen)

    def near(value, *shape, s=0.1):
        return torch.full(shape, float(value), dtype=dtype, device=device) + mat(*shape, s=s)

    st = {"embed": mat(cfg.vocab_size, W), "head": mat(cfg.vocab_size, W, s=W ** -0.5), "final.norm": near(1.0, W)}
    if spec.bigram is not None:
        st["bigram"] = mat(spec.bigram.buckets + 1, W, s=0.5)
    for i, L in enumerate(spec.layers):
        p, m, q = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        st[p + "norm1"] = near(1.0, W)
        if L.kind == "attention":
            A = L.battn
            st[m + "q"], st[m + "k"] = mat(A.heads * A.dim, W, s=W ** -0.5), mat(A.kv_heads * A.dim, W, s=W ** -0.5)
            st[m + "q.norm"], st[m + "k.norm"] = near(1.0, A.dim), near(1.0, A.dim)
            st[m + "r1"], st[m + "r2"] = near(0.5, A.heads, s=0.2).abs(), near(0.3, A.heads, s=0.1).abs()
            st[m + "g"] = mat(A.heads * A.vdim, W, s=W ** -0.5)
            st[m + "o"] = mat(W, A.heads * A.vdim, s=(A.heads * A.vdim) ** -0.5)
        else:
            C = L.gru.width
            for n in "zxg":
                st[m + n] = mat(C, W, s=W ** -0.5)
            st[m + "z.b"], st[m + "x.b"] = mat(C, s=0.5), mat(C, s=0.5)
            st[m + "o"] = mat(W, C, s=C ** -0.5)
        if L.ff:
            st[p + "norm2"] = near(1.0, W)
            st[q + "up"], st[q + "down"] = mat(L.ff, W, s=W ** -0.5), mat(W, L.ff, s=L.ff ** -0.5)
        elif L.moe is not None:
            M = L.moe
            st[p + "norm2"] = near(1.0, W)
            st[q + "router"], st[q + "correction"] = mat(M.outputs, W, s=W ** -0.5), mat(M.outputs, s=0.05)
            for e in range(M.experts):
                st[f"{q}e{e}.gate"], st[f"{q}e{e}.up"] = mat(M.ff, W, s=W ** -0.5), mat(M.ff, W, s=W ** -0.5)
                st[f"{q}e{e}.down"] = mat(W, M.ff, s=M.ff ** -0.5)
            if M.shared_ff:
                st[q + "shared.gate"], st[q + "shared.up"] = mat(M.shared_ff, W, s=W ** -0.5), mat(M.shared_ff, W, s=W ** -0.5)
                st[q + "shared.down"], st[q + "shared.sg"] = mat(W, M.shared_ff, s=M.shared_ff ** -0.5), mat(1, W, s=W ** -0.5)
    return st


def sandwich_synthetic_state(cfg: ModelConfig, seed: int = 0, decay_rank: int = 64, device="cpu",
                             dtype=torch.float32) -> dict:
    """Seeded random tensors under a Tativik checkpoint's names (benchmarks and tests: nothing can be
    downloaded).  `decay_rank`: the inner width of the low-rank decay projection."""
    spec, W = cfg.hybrid, cfg.hidden_size
    gen = torch.Generator(device=device).manual_seed(seed)

    def mat(*shape, s=1.0):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, s, generator=gen)

    def near(value, *shape, s=0.1):
        return torch.full(shape, float(value), dtype=dtype, device=device) + mat(*shape, s=s)

    st = {"embed": mat(cfg.vocab_size, W), "embed.norm": near(1.0, W), "head": mat(cfg.vocab_size, W, s=W ** -0.5),
          "final.norm": near(1.0, W)}
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", f"l{i}.mix."
        st[p + "norm1"], st[p + "norm1b"] = near(1.0, W), near(1.0, W)
        st[p + "rg1"], st[p + "rg1.b"] = mat(W, W, s=W ** -0.5), mat(W, s=0.5)
        if L.kind == "general_delta":
            C = L.gdelta.heads * L.gdelta.dim
            for n in "rkvga":
                st[m + n] = mat(C, W, s=W ** -0.5)
            st[m + "a.b"], st[m + "w0"], st[m + "norm"] = mat(C, s=0.5), mat(C), near(1.0, C)
            st[m + "w1"], st[m + "w2"] = mat(decay_rank, W, s=W ** -0.5), mat(C, decay_rank, s=decay_rank ** -0.5)
            st[m + "o"] = mat(W, C, s=C ** -0.5)
        else:
            A = L.lattn
            st[m + "dq"], st[m + "dq.norm"] = mat(A.q_rank, W, s=W ** -0.5), near(1.0, A.q_rank)
            st[m + "uq"] = mat(A.heads * (A.dim + A.rot_dim), A.q_rank, s=A.q_rank ** -0.5)
            if A.kv_from is None:
                st[m + "dkv"], st[m + "dkv.norm"] = mat(A.kv_rank + A.rot_dim, W, s=W ** -0.5), near(1.0, A.kv_rank)
            st[m + "uk"] = mat(A.heads * A.dim, A.kv_rank, s=A.kv_rank ** -0.5)
            st[m + "uv"] = mat(A.heads * A.vdim, A.kv_rank, s=A.kv_rank ** -0.5)
            st[m + "sink"], st[m + "g"] = mat(A.heads), mat(A.heads, W, s=W ** -0.5)
            st[m + "o"] = mat(W, A.heads * A.vdim, s=(A.heads * A.vdim) ** -0.5)
        if L.moe is not None:
            M, q = L.moe, p + "mlp."
            st[p + "norm2"], st[p + "norm2b"] = near(1.0, W), near(1.0, W)
            st[p + "rg2"], st[p + "rg2.b"] = mat(W, W, s=W ** -0.5), mat(W, s=0.5)
            st[q + "router"], st[q + "correction"] = mat(M.experts, W, s=W ** -0.5), mat(M.experts, s=0.3)
            for e in range(M.experts):
                st[f"{q}e{e}.gate"], st[f"{q}e{e}.up"] = mat(M.ff, W, s=W ** -0.5), mat(M.ff, W, s=W ** -0.5)
                st[f"{q}e{e}.down"] = mat(W, M.ff, s=M.ff ** -0.5)
    return st


def hybrid_synthetic_state(cfg: ModelConfig, seed: int = 0, std: float = 0.02, rank: int = 32, device="cpu",
                           dtype=torch.float32) -> dict:
    """Seeded random tensors under a Lozupel checkpoint's names (benchmarks and tests: nothing can be
    downloaded).  `rank`: the inner width of the low-rank decay / gate projections."""
    spec, W = cfg.hybrid, cfg.hidden_size
    if spec.arrangement == "sandwich":
        return sandwich_synthetic_state(cfg, seed=seed, device=device, dtype=dtype)
    if cfg.architecture == "Tafisun":
        return tafisun_synthetic_state(cfg, seed=seed, device=device, dtype=dtype)
    if spec.arrangement == "parallel":
        return bemulorn_synthetic_state(cfg, seed=seed, device=device, dtype=dtype)
    gen = torch.Generator(device=device).manual_seed(seed)

    def mat(*shape, s=std):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, s, generator=gen)

    def near(value, *shape, s=0.1):
        return torch.full(shape, float(value), dtype=dtype, device=device) + mat(*shape, s=s)

    st = {"embed": mat(cfg.vocab_size, W, s=1.0), "head": mat(cfg.vocab_size, W), "final.norm": near(1.0)}
    if spec.loop_times > 0:
        st["loop.step"] = mat(spec.loop_times, W, s=0.1)
    for i, L in enumerate(spec.layers):
        p = f"l{i}."
        st[p + "norm1"] = near(1.0)
        m = p + "mix." + ("right." if L.kind == "parallel" else "")
        D = L.delta
        qk, vv = D.kv_heads * D.dim, D.heads * D.vdim
        for n, c in (("q", qk), ("k", qk), ("v", vv)):
            st[m + n] = mat(c, W, s=W ** -0.5)
            st[m + n + ".conv"] = mat(c, D.conv, s=D.conv ** -0.5)
        st[m + "b"] = mat(D.heads, W, s=W ** -0.5)
        st[m + "A_log"] = mat(D.heads, s=0.5)
        st[m + "norm"] = near(1.0, D.vdim)
        st[m + "o"] = mat(W, vv, s=vv ** -0.5)
        if D.per_channel:
            st[m + "a1"], st[m + "a2"] = mat(rank, W, s=W ** -0.5), mat(D.heads * D.dim, rank, s=rank ** -0.5)
            st[m + "g1"], st[m + "g2"] = mat(rank, W, s=W ** -0.5), mat(vv, rank, s=rank ** -0.5)
            st[m + "dt_bias"] = mat(D.heads * D.dim, s=0.5)
        else:
            st[m + "a"], st[m + "g"] = mat(D.heads, W, s=W ** -0.5), mat(vv, W, s=W ** -0.5)
            st[m + "dt_bias"] = mat(D.heads, s=0.5)
        if L.kind == "parallel":
            A, a = L.attn, p + "mix.left."
            st[a + "q"], st[a + "k"] = mat(A.heads * A.dim, W, s=W ** -0.5), mat(A.kv_heads * A.dim, W, s=W ** -0.5)
            st[a + "v"], st[a + "g"] = mat(A.kv_heads * A.vdim, W, s=W ** -0.5), mat(A.heads, W, s=W ** -0.5)
            st[a + "temp"], st[a + "pb"] = near(1.0, A.heads), near(-2.0, A.heads, s=0.5)
            st[a + "o"] = mat(W, A.heads * A.vdim, s=(A.heads * A.vdim) ** -0.5)
            st[a + "out"], st[m + "out"] = near(1.0, W), near(1.0, W)
        if L.ff:
            st[p + "norm2"] = near(1.0)
            st[p + "mlp.gate"], st[p + "mlp.up"] = mat(L.ff, W, s=W ** -0.5), mat(L.ff, W, s=W ** -0.5)
            st[p + "mlp.down"] = mat(W, L.ff, s=L.ff ** -0.5)
    return st


def from_state_dict(cfg, state: dict, dtype, device, **kw) -> ModelWeights:
    def get(name):
        t = state[name]
        return t if isinstance(t, torch.Tensor) else torch.from_numpy(t)
    return from_getter(cfg, get, dtype, device, **kw)


def has_checkpoint(model_dir: str) -> bool:
    return os.path.isdir(model_dir) and bool(glob.glob(os.path.join(model_dir, "*.safetensors")))


def from_safetensors(cfg, model_dir: str, dtype, device, **kw) -> ModelWeights:
    from safetensors import safe_open

    index = os.path.join(model_dir, "model.safetensors.index.json")
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    where = {}
    if os.path.isfile(index):
        with open(index) as f:
            where = {k: os.path.join(model_dir, v) for k, v in json.load(f)["weight_map"].items()}
    handles = {}

    def get(name):
        path = where.get(name)
        if path is None:
            for fpath in files:
                h = handles.setdefault(fpath, safe_open(fpath, framework="pt", device="cpu"))
                if name in h.keys():
                    path = fpath
                    break
            else:
                raise KeyError(f"{name} not found in {model_dir}")
        h = handles.setdefault(path, safe_open(path, framework="pt", device="cpu"))
        return h.get_tensor(name)

    return from_getter(cfg, get, dtype, device, **kw)


def synthetic(cfg: ModelConfig, dtype, device, seed: int = 0, tp_rank: int = 0, tp_size: int = 1,
              num_layers: Optional[int] = None, std: float = 0.02, shard_mlp: bool = False,
              shard_vocab: bool = False) -> ModelWeights:
    """Seeded N(0, std^2) matrices of the real shapes, generated on the device
    (an 8B model is 15 GB: too slow to draw on the host).  Every rank draws the
    replicated tensors from the same stream so they are bit-identical across ranks."""
    if cfg.family == "opt":
        return _opt_synthetic(cfg, dtype, device, seed, tp_size, num_layers, std)
    if cfg.family == "hybrid":
        _hybrid_one_gpu(tp_size, num_layers)
        state = hybrid_synthetic_state(cfg, seed=seed, device=device)
        w = from_state_dict(cfg, state, dtype, device)
        w.synthetic = True
        return w
    nh_l, nkv_l, _, _ = _shard_heads(cfg, tp_rank, tp_size)
    H, F, V, d = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.head_dim
    if shard_mlp:
        fs = _shard_mlp(cfg, tp_rank, tp_size)
        F = fs.stop - fs.start
    shared = torch.Generator(device=device).manual_seed(seed)
    local = torch.Generator(device=device).manual_seed(seed * 1000003 + 17 + tp_rank)

    def mat(gen, *shape):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0.0, std, generator=gen)

    L = num_layers if num_layers is not None else cfg.num_hidden_layers
    w = ModelWeights(embed=mat(shared, V, H), synthetic=True)
    for _ in range(L):
        w.layers.append(LayerWeights(
            qkv_w=mat(local, (nh_l + 2 * nkv_l) * d, H),
            qkv_b=mat(local, (nh_l + 2 * nkv_l) * d) if cfg.attention_bias else None,
            o_w=mat(local, H, nh_l * d),
            gate_up_w=mat(local if shard_mlp else shared, 2 * F, H),
            down_w=mat(local if shard_mlp else shared, H, F),
            input_norm=torch.ones(H, dtype=dtype, device=device),
            post_norm=torch.ones(H, dtype=dtype, device=device)))
    w.final_norm = torch.ones(H, dtype=dtype, device=device)
    if shard_vocab:
        vs = _shard_vocab(cfg, tp_rank, tp_size)
        w.lm_head = w.embed[vs] if cfg.tie_word_embeddings else mat(local, vs.stop - vs.start, H)
    else:
        w.lm_head = w.embed if cfg.tie_word_embeddings else mat(shared, V, H)
    return w
