"""Model and engine configuration.

``EngineArgs`` mirrors the engine CLI the reference harness generates
(benchmark-vllm/vllm_templates.py:50-87, vllm_manager.py:399-416): same flag
names and defaults as the engine it launches, so a `VLLMConfig`
(benchmark-vllm/models.py:5-31) maps onto it field by field.
``ModelConfig`` is read from the HF-style ``config.json`` of a local model
directory (weights are served from a local path, benchmark-mlflow/vllm_processor.py:29).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Optional

SUPPORTED_ARCHS = ("LlamaForCausalLM", "Qwen2ForCausalLM", "MistralForCausalLM", "OPTForCausalLM", "Lozupel", "Tativik", "Tafisun", "Bemulorn")

# Well-known geometries, used when --model names one of them and no local
# config.json exists (synthetic-weight benchmarking; there is no network).
KNOWN_MODELS = {
    "llama-3-8b": dict(architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=4096,
                       intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                       num_key_value_heads=8, rope_theta=500000.0, rms_norm_eps=1e-5,
                       max_position_embeddings=8192, tie_word_embeddings=False, torch_dtype="bfloat16"),
    "llama-3-70b": dict(architectures=["LlamaForCausalLM"], vocab_size=128256, hidden_size=8192,
                        intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64,
                        num_key_value_heads=8, rope_theta=500000.0, rms_norm_eps=1e-5,
                        max_position_embeddings=8192, tie_word_embeddings=False, torch_dtype="bfloat16"),
    # the model the harness launches when a request names none (benchmark-vllm/models.py:7)
    "opt-125m": dict(architectures=["OPTForCausalLM"], vocab_size=50272, hidden_size=768, ffn_dim=3072,
                     num_hidden_layers=12, num_attention_heads=12, max_position_embeddings=2048,
                     word_embed_proj_dim=768, do_layer_norm_before=True, activation_function="relu",
                     bos_token_id=2, eos_token_id=2, torch_dtype="float16"),      # published in float16
    "qwen2-7b": dict(architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584,
                     intermediate_size=18944, num_hidden_layers=28, num_attention_heads=28,
                     num_key_value_heads=4, rope_theta=1000000.0, rms_norm_eps=1e-6,
                     max_position_embeddings=32768, tie_word_embeddings=False, torch_dtype="bfloat16"),
}


def _known_key(name: str) -> Optional[str]:
    n = os.path.basename(name.rstrip("/")).lower().replace("meta-", "").replace("_", "-")
    for key in KNOWN_MODELS:
        if key in n or key.replace("-", "") in n.replace("-", ""):
            return key
    return None


@dataclass
class WindowAttnSpec:
    """Sliding-window attention with sigmoid weights: sigmoid(q.k * scale * temp[h] + bias[h]) for the
    keys j with 0 <= i - j < window, not normalised over keys; rotary positions on the first rot_dims
    coordinates of each head; one output gate per head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    rot_dims: int
    rot_base: float
    scale: float


@dataclass
class DeltaSpec:
    """Gated delta rule mixer: heads value heads of vdim channels on kv_heads query / key heads of dim
    channels, a causal convolution of `conv` taps on q, k and v.  per_channel: one decay per key
    channel (projected through a low-rank pair, as is the output gate, which is then a sigmoid)
    instead of one per head (full-rank projections, SiLU gate)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    per_channel: bool = False


@dataclass
class GeneralDeltaSpec:
    """General delta rule mixer: per head a state [dim, dim] with a decay per key channel (projected
    through a low-rank pair with a tanh between) and a removal along the unit key at a rate per key
    channel; receptance, key and value all heads x dim; output normed per head and gated."""
    heads: int
    dim: int


@dataclass
class LatentAttnSpec:
    """Softmax attention through low-rank latents: queries through q_rank, keys and values through
    kv_rank; per head `dim` unrotated and `rot_dim` rotated query / key coordinates (the rotated key
    part is one vector shared by all heads, rotation on its first rot_dims coordinates), values of
    vdim; sliding window; a learned sink per head in the softmax denominator; one output gate per
    head.  kv_from: the layer whose cached latent and rotated key this layer reads instead of making
    its own (None: its own).  q_rank 0: not in the configuration, the weights' shape gives it; a
    configuration without a window gets one longer than any sequence."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    window: int
    rot_dims: int
    rot_base: float
    scale: float
    kv_from: Optional[int] = None


@dataclass
class MoESpec:
    """Mixture of experts: `top` of `experts` gated feed-forwards of width ff per token, scored by
    sigmoid(router), chosen by score + correction inside the best `keep` of `groups` groups of
    neighbouring experts, weighted by the score itself."""
    experts: int
    top: int
    groups: int
    keep: int
    ff: int
    # what follows defaults to the first design that used this spec
    score: str = "sigmoid"                  # "sigmoid": each expert by itself; "softmax": over all router outputs;
                                            # "chosen_softmax": choice by the logits, weights a softmax over the chosen alone
    router_bias: bool = False               # the router logits carry a learned bias
    shared_gated: bool = True               # the shared expert is scaled by a sigmoid of one projected number per token
    group_score: str = "top2"               # a group scores the sum of its two best choice scores, or ("max") its best
    weight_scale: float = 1.0               # the chosen experts' scores are multiplied by this
    identity: int = 0                       # router outputs past `experts` that stand for "the input itself"; groups
                                            # are formed over experts and identity outputs together
    limit: Optional[float] = None           # None: silu(g) * u.  A number: g = min(g, limit), u = clamp(u, -limit, limit),
                                            # g * sigmoid(1.702 g) * (u + 1)
    shared_ff: int = 0                      # width of an expert that every token uses, scaled by a sigmoid of one
    shared_limit: Optional[float] = None    # projected number per token; 0: none

    @property
    def outputs(self) -> int:
        """Router outputs: experts and identity experts."""
        return self.experts + self.identity

    def check(self, where: str) -> None:
        n = self.outputs
        if self.experts < 1 or self.identity < 0 or n % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * (n // self.groups):
            raise ValueError(f"{where}: {self.experts} experts + {self.identity} identity in {self.groups} groups, "
                             f"{self.keep} kept, {self.top} chosen do not fit")


@dataclass
class BlockAttnSpec:
    """Softmax attention inside blocks of `block` positions (position i sees j <= i with
    i // block == j // block; block 0: plain causal), grouped heads, no rotation: the score is
    q.k * scale - r1[h] * ln(1 + r2[h] * (i - j)).  Queries and keys get an RMS norm per head with one
    weight vector shared by the heads.  values_are_keys: no value projection exists; the key
    projection, taken ahead of its norm, doubles as the value (then vdim == dim).  The concatenated heads are
    multiplied by a sigmoid gate of their own width.

    What follows the first design's fields switches its particulars off and others on: qk_norm /
    penalty False: plain q.k * scale; rot_dims > 0: rotary positions on the first rot_dims coordinates
    of every query and key head (coordinate i paired with i + rot_dims / 2), frequencies blended for
    longer contexts by rot_scaling; bias: q, k and v projections carry biases; sink: the softmax
    denominator holds one more term exp(sink) that carries no value; gate_per_head: the gate is one
    number per head; kv_from: the layer has no key / value projections and attends to the pages of
    that earlier layer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    block: int
    scale: float
    values_are_keys: bool = True
    qk_norm: bool = True
    penalty: bool = True
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional["RotaryScaling"] = None
    bias: bool = False
    sink: Optional[float] = None
    gate_per_head: bool = False
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class RotaryScaling:
    """Blend of rotary frequencies for contexts longer than `original` positions: with
    c(r) = dims * ln(original / (2 pi r)) / (2 ln base), lo = max(floor(c(fast)), 0),
    hi = min(ceil(c(slow)), dims - 1) and m_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at
    f_i / factor * m_i + f_i * (1 - m_i); cos and sin are both multiplied by 0.1 ln(factor) + 1."""
    factor: float
    original: float
    fast: float
    slow: float

    def frequencies(self, rot_dims: int, base: float):
        """(float64 frequencies [rot_dims / 2], the factor on cos and sin)."""
        import math
        import numpy as np
        i = np.arange(rot_dims // 2, dtype=np.float64)
        f = float(base) ** (-2.0 * i / rot_dims)

        def c(r):
            return rot_dims * math.log(self.original / (2.0 * math.pi * r)) / (2.0 * math.log(base))
        lo, hi = max(math.floor(c(self.fast)), 0), min(math.ceil(c(self.slow)), rot_dims - 1)
        m = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / self.factor * m + f * (1.0 - m), 0.1 * math.log(self.factor) + 1.0


@dataclass
class MinGRUSpec:
    """Gated recurrence over `width` channels whose gates read only the current token:
    S <- (1 - z) S + z c, z = sigmoid(.), c = u + 1/2 for u >= 0 and sigmoid(u) below; the output is
    S * silu(gate), projected."""
    width: int


@dataclass
class BigramSpec:
    """A second embedding table indexed by a hash of the previous and the current token:
    row (prev * mul_prev + cur * mul_cur) mod buckets; the first token of a sequence takes row `buckets`."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class HybridLayerSpec:
    # "delta": one DeltaSpec; "parallel": window attention beside a delta mixer;
    # "general_delta": one GeneralDeltaSpec; "latent_attention": one LatentAttnSpec
    kind: str
    delta: DeltaSpec = None
    attn: Optional[WindowAttnSpec] = None
    ff: Optional[int] = None                # width of the dense gated feed-forward, None: the layer has none
    gdelta: Optional[GeneralDeltaSpec] = None
    lattn: Optional[LatentAttnSpec] = None
    moe: Optional[MoESpec] = None           # a mixture-of-experts feed-forward instead of a dense one
    battn: Optional[BlockAttnSpec] = None   # kind "attention"
    gru: Optional[MinGRUSpec] = None        # kind "mingru"
    ff_act: str = "gelu_gated"              # the dense feed-forward: gelu_tanh(gate) * up, or "relu2": relu(up)^2, no gate,
                                            # or "limited": g' sigmoid(1.702 g') (u' + 1), g' = min(g, ff_limit),
                                            # u' = clamp(u, -ff_limit, ff_limit)
    ff_limit: Optional[float] = None


@dataclass
class HybridSpec:
    """A decoder whose layers each name their sequence mixer, with an optional weight-shared loop:
    layers loop_start .. loop_stop - 1 run loop_times times in a row (separate cache and state per
    pass); before every pass a learned vector is added to the residual, and before every pass but
    the first the embedding output too."""
    layers: list
    embed_scale: float = 1.0
    logit_softcap: Optional[float] = None
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0                     # 0: no loop
    # "pre": x += sublayer(norm(x)), norms with one learned number.  "sandwich": the embedding is
    # normed, and x += residual_mult * norm_b(sublayer(h) * sigmoid(Wg h + bg)) with h = norm(x);
    # every such norm is an RMS norm in norm_groups equal parts with a weight vector.  "parallel":
    # x += mixer(h) + ff(h) with h = norm(x): one norm per layer, both sub-layers read it
    arrangement: str = "pre"
    norm_groups: int = 1
    residual_mult: float = 1.0
    norm_vector: bool = False               # "pre" arrangement: norms carry a weight per channel instead of one number
    bigram: Optional[BigramSpec] = None     # a hashed previous-token embedding is added (the previous token is state)
    sinusoid_base: float = 0.0              # > 0: sin / cos of pos * base^(-2i / width) in entries 2i / 2i + 1 is added
    learned_positions: bool = False         # a learned vector per position is added to the scaled embedding
    logit_scale: float = 1.0                # the logits are multiplied by this

    def runs(self):
        """[(layer index, pass number or None)] in execution order: one cache / state each."""
        n = len(self.layers)
        if self.loop_times <= 0:
            return [(i, None) for i in range(n)]
        out = [(i, None) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            out += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, None) for i in range(self.loop_stop, n)]

    @classmethod
    def from_bemulorn(cls, d: dict) -> "HybridSpec":
        layers = []
        for i, spec in enumerate(d["layers"]):
            m, mlp = spec["mixer"], spec.get("mlp")
            kw = {}
            if mlp is not None and mlp.get("kind", "dense") == "dense":
                kw.update(ff=int(mlp["ff"]), ff_act="limited", ff_limit=float(mlp["limit"]))
            elif mlp is not None and mlp.get("kind") == "moe":
                r, sh = mlp["router"], mlp.get("shared") or None
                moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), groups=1, keep=1, ff=int(mlp["expert"]["ff"]),
                              score="chosen_softmax", router_bias=True, shared_ff=int(sh["ff"]) if sh else 0,
                              shared_gated=False)
                moe.check(f"layer {i}")
                kw.update(moe=moe)
            elif mlp is not None:
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not supported (dense, moe)")
            if spec["type"] != "attention":
                raise ValueError(f"layer type {spec['type']!r} is not supported (attention)")
            rot = m.get("rot") or {}
            sc = rot.get("scaling") or None
            a = BlockAttnSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                              vdim=int(m.get("vdim", m["dim"])), block=int((m.get("mask") or {}).get("size") or 0),
                              scale=float(m["scale"]), values_are_keys=False, qk_norm=False, penalty=False,
                              rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                              rot_scaling=RotaryScaling(float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                                        float(sc["slow"])) if sc else None,
                              bias=True, sink=0.0, gate_per_head=True,
                              kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None else None))
            if a.heads < 1 or a.kv_heads < 1 or a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: kv_heads {a.kv_heads} must divide heads {a.heads}")
            if a.rot_dims > a.dim or a.rot_dims % 2:
                raise ValueError(f"layer {i}: {a.rot_dims} rotated coordinates do not fit heads of {a.dim}")
            if a.kv_from is not None:
                src = layers[a.kv_from].battn if 0 <= a.kv_from < i else None
                if src is None or src.kv_from is not None:
                    raise ValueError(f"layer {i}: kv_from {a.kv_from} must name an earlier attention layer that has "
                                     "key and value projections of its own")
                if (src.kv_heads, src.dim, src.vdim, src.rot_dims, src.rot_base, src.rot_scaling) != \
                        (a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base, a.rot_scaling):
                    raise ValueError(f"layer {i}: key / value heads and rotation differ from layer {a.kv_from}'s")
            layers.append(HybridLayerSpec("attention", battn=a, **kw))
        return cls(layers=layers, arrangement="parallel", norm_vector=True, learned_positions=True,
                   embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(d.get("logit_scale", 1.0)))

    @classmethod
    def from_tafisun(cls, d: dict) -> "HybridSpec":
        layers = []
        for i, spec in enumerate(d["layers"]):
            m, mlp = spec["mixer"], spec.get("mlp")
            kw = {}
            if mlp is not None and mlp.get("kind", "dense") == "dense":
                kw.update(ff=int(mlp["ff"]), ff_act="relu2")
            elif mlp is not None and mlp.get("kind") == "moe":
                r, sh = mlp["router"], mlp.get("shared") or None
                g = r.get("groups") or {"count": 1, "keep": 1}
                moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), groups=int(g.get("count", 1)),
                              keep=int(g.get("keep", g.get("count", 1))), ff=int(mlp["expert"]["ff"]), score="softmax",
                              group_score="max", weight_scale=float(r.get("scale", 1.0)), identity=int(r.get("identity", 0)),
                              limit=float(mlp["expert"]["limit"]), shared_ff=int(sh["ff"]) if sh else 0,
                              shared_limit=float(sh["limit"]) if sh else None)
                moe.check(f"layer {i}")
                kw.update(moe=moe)
            elif mlp is not None:
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not supported (dense, moe)")
            if spec["type"] == "attention":
                a = BlockAttnSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                  vdim=int(m.get("vdim", m["dim"])), block=int((m.get("mask") or {}).get("size") or 0),
                                  scale=float(m["scale"]))
                if a.heads < 1 or a.kv_heads < 1 or a.heads % a.kv_heads:
                    raise ValueError(f"layer {i}: kv_heads {a.kv_heads} must divide heads {a.heads}")
                if a.vdim != a.dim:
                    raise ValueError(f"layer {i}: the values are the keys, so vdim {a.vdim} must equal dim {a.dim}")
                layers.append(HybridLayerSpec("attention", battn=a, **kw))
            elif spec["type"] == "mingru":
                layers.append(HybridLayerSpec("mingru", gru=MinGRUSpec(int(m["width"])), **kw))
            else:
                raise ValueError(f"layer type {spec['type']!r} is not supported (attention, mingru)")
        b = (d.get("embedding") or {}).get("bigram")
        return cls(layers=layers, norm_vector=True, sinusoid_base=10000.0,
                   bigram=BigramSpec(int(b["buckets"]), int(b["mul_prev"]), int(b["mul_cur"])) if b else None)

    @classmethod
    def from_tativik(cls, d: dict) -> "HybridSpec":
        layers = []
        for i, spec in enumerate(d["layers"]):
            m, mlp = spec["mixer"], spec.get("mlp")
            moe = None
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not supported (moe)")
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), groups=int(g["count"]), keep=int(g["keep"]),
                              ff=int(mlp["expert"]["ff"]))
                if moe.experts % moe.groups or not 1 <= moe.keep <= moe.groups \
                        or not 1 <= moe.top <= moe.keep * (moe.experts // moe.groups):
                    raise ValueError(f"layer {i}: {moe.experts} experts in {moe.groups} groups, {moe.keep} kept, "
                                     f"{moe.top} chosen do not fit")
            if spec["type"] == "general_delta":
                layers.append(HybridLayerSpec("general_delta", gdelta=GeneralDeltaSpec(int(m["heads"]), int(m["dim"])),
                                              moe=moe))
            elif spec["type"] == "latent_attention":
                rot = m.get("rot") or {}
                a = LatentAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                                   kv_rank=int(m["kv_rank"]), q_rank=int(m.get("q_rank") or 0),
                                   window=int((m.get("mask") or {}).get("size") or 1 << 30),
                                   rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot.get("base", 10000.0)),
                                   scale=float(m["scale"]),
                                   kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None else None))
                if a.rot_dims > a.rot_dim or a.rot_dims % 2:
                    raise ValueError(f"layer {i}: {a.rot_dims} rotated coordinates do not fit rot_dim {a.rot_dim}")
                if a.kv_from is not None:
                    src = layers[a.kv_from].lattn if 0 <= a.kv_from < i else None
                    if src is None or src.kv_from is not None:
                        raise ValueError(f"layer {i}: kv_from {a.kv_from} must name an earlier latent attention "
                                         "layer that makes its own latent")
                    if (src.kv_rank, src.rot_dim, src.rot_dims, src.rot_base) != (a.kv_rank, a.rot_dim, a.rot_dims, a.rot_base):
                        raise ValueError(f"layer {i}: latent sizes and rotation differ from layer {a.kv_from}'s")
                layers.append(HybridLayerSpec("latent_attention", lattn=a, moe=moe))
            else:
                raise ValueError(f"layer type {spec['type']!r} is not supported (general_delta, latent_attention)")
        return cls(layers=layers, arrangement="sandwich", norm_groups=int(d["norm"].get("groups", 1)),
                   residual_mult=float(d.get("residual_mult", 1.0)))

    @classmethod
    def from_lozupel(cls, d: dict) -> "HybridSpec":
        def delta(m, per_channel):
            return DeltaSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                             vdim=int(m["vdim"]), conv=int(m["conv"]), per_channel=per_channel)
        layers = []
        for spec in d["layers"]:
            m, mlp = spec["mixer"], spec.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is not supported (dense)")
            ff = int(mlp["ff"]) if mlp is not None else None
            if spec["type"] == "delta":
                layers.append(HybridLayerSpec("delta", delta=delta(m, False), ff=ff))
            elif spec["type"] == "parallel":
                a = m["left"]
                attn = WindowAttnSpec(heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]),
                                      vdim=int(a["vdim"]), window=int(a["mask"]["size"]),
                                      rot_dims=int(a["rot"]["dims"]), rot_base=float(a["rot"]["base"]),
                                      scale=float(a["scale"]))
                layers.append(HybridLayerSpec("parallel", delta=delta(m["right"], True), attn=attn, ff=ff))
            else:
                raise ValueError(f"layer type {spec['type']!r} is not supported (delta, parallel)")
        for L in layers:
            for m in (L.delta, L.attn):
                if m is not None and (m.heads % m.kv_heads or m.heads < 1):
                    raise ValueError(f"kv_heads {m.kv_heads} must divide heads {m.heads}")
        loop = d.get("loop") or {}
        out = cls(layers=layers, embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  logit_softcap=(float(d["logit_softcap"]) if d.get("logit_softcap") else None),
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 0)))
        if out.loop_times > 0 and not 0 <= out.loop_start < out.loop_stop <= len(layers):
            raise ValueError(f"loop {out.loop_start}..{out.loop_stop} does not fit {len(layers)} layers")
        return out


@dataclass
class ModelConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rope_theta: float
    rope_scaling: Optional[dict]
    rms_norm_eps: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    attention_bias: bool
    bos_token_id: Optional[int] = None
    eos_token_id: Any = None
    # the decoder family: "llama" (RMSNorm, rotary positions, SwiGLU MLP) or "opt" (LayerNorm with
    # bias, learned positions stored at an offset, biased projections, fc1 -> ReLU -> fc2)
    family: str = "llama"
    position_offset: int = 0
    # the type the checkpoint's weights are stored in (config.json's torch_dtype / dtype), if it says
    torch_dtype: Optional[str] = None
    # family "hybrid": the per-layer mixers, loop and output constants; the Llama-shaped fields above
    # then hold the width, the vocabulary and the largest head geometry for sizing only
    hybrid: Optional[HybridSpec] = None

    @classmethod
    def _from_lozupel_dict(cls, d: dict) -> "ModelConfig":
        spec = HybridSpec.from_lozupel(d)
        mixers = [m for L in spec.layers for m in (L.attn, L.delta) if m is not None]
        return cls(architecture="Lozupel", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                   intermediate_size=max([L.ff or 0 for L in spec.layers] + [0]), num_hidden_layers=len(spec.layers),
                   num_attention_heads=max(m.heads for m in mixers), num_key_value_heads=max(m.kv_heads for m in mixers),
                   head_dim=max(m.dim for m in mixers), rope_theta=0.0, rope_scaling=None,
                   rms_norm_eps=float(d["norm"]["eps"]), max_position_embeddings=int(d.get("max_positions", 1 << 17)),
                   tie_word_embeddings=False, attention_bias=False, bos_token_id=d.get("bos_token_id"),
                   eos_token_id=d.get("eos_token_id"), family="hybrid", hybrid=spec)

    @classmethod
    def _from_tafisun_dict(cls, d: dict) -> "ModelConfig":
        spec = HybridSpec.from_tafisun(d)
        att = [L.battn for L in spec.layers if L.battn is not None]
        ffs = [L.ff or 0 for L in spec.layers] + [max(L.moe.ff, L.moe.shared_ff) for L in spec.layers if L.moe] + [0]
        return cls(architecture="Tafisun", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                   intermediate_size=max(ffs), num_hidden_layers=len(spec.layers),
                   num_attention_heads=max([a.heads for a in att] + [1]), num_key_value_heads=max([a.kv_heads for a in att] + [1]),
                   head_dim=max([a.dim for a in att] + [1]), rope_theta=0.0, rope_scaling=None,
                   rms_norm_eps=float(d["norm"]["eps"]), max_position_embeddings=int(d.get("max_positions", 1 << 17)),
                   tie_word_embeddings=False, attention_bias=False, bos_token_id=d.get("bos_token_id"),
                   eos_token_id=d.get("eos_token_id"), family="hybrid", hybrid=spec)

    @classmethod
    def _from_bemulorn_dict(cls, d: dict) -> "ModelConfig":
        spec = HybridSpec.from_bemulorn(d)
        att = [L.battn for L in spec.layers]
        ffs = [L.ff or 0 for L in spec.layers] + [max(L.moe.ff, L.moe.shared_ff) for L in spec.layers if L.moe] + [0]
        return cls(architecture="Bemulorn", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                   intermediate_size=max(ffs), num_hidden_layers=len(spec.layers),
                   num_attention_heads=max([a.heads for a in att] + [1]), num_key_value_heads=max([a.kv_heads for a in att] + [1]),
                   head_dim=max([a.dim for a in att] + [1]), rope_theta=0.0, rope_scaling=None,
                   rms_norm_eps=float(d["norm"]["eps"]), max_position_embeddings=int(d.get("max_positions", 1 << 17)),
                   tie_word_embeddings=False, attention_bias=True, bos_token_id=d.get("bos_token_id"),
                   eos_token_id=d.get("eos_token_id"), family="hybrid", hybrid=spec)

    @classmethod
    def _from_tativik_dict(cls, d: dict) -> "ModelConfig":
        spec = HybridSpec.from_tativik(d)
        if int(d["width"]) % spec.norm_groups:
            raise ValueError(f"width {d['width']} is not a multiple of {spec.norm_groups} norm groups")
        heads = [m.heads for L in spec.layers for m in (L.gdelta, L.lattn) if m is not None]
        dims = [L.gdelta.dim if L.gdelta is not None else L.lattn.dim + L.lattn.rot_dim for L in spec.layers]
        return cls(architecture="Tativik", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                   intermediate_size=max([L.moe.ff if L.moe else 0 for L in spec.layers] + [0]),
                   num_hidden_layers=len(spec.layers), num_attention_heads=max(heads), num_key_value_heads=1,
                   head_dim=max(dims), rope_theta=0.0, rope_scaling=None, rms_norm_eps=float(d["norm"]["eps"]),
                   max_position_embeddings=int(d.get("max_positions", 1 << 17)), tie_word_embeddings=False,
                   attention_bias=False, bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"),
                   family="hybrid", hybrid=spec)

    @classmethod
    def _from_opt_dict(cls, d: dict) -> "ModelConfig":
        H, nh = d["hidden_size"], d["num_attention_heads"]
        if d.get("word_embed_proj_dim", H) != H:
            raise ValueError("OPT checkpoints whose embeddings are projected (word_embed_proj_dim != hidden_size, "
                             "opt-350m) are not supported")
        if not d.get("do_layer_norm_before", True):
            raise ValueError("OPT checkpoints that normalise after the sub-layers (do_layer_norm_before false, "
                             "opt-350m) are not supported")
        if d.get("activation_function", "relu") != "relu" or not d.get("enable_bias", True) \
                or not d.get("layer_norm_elementwise_affine", True):
            raise ValueError("OPT variants without biases / affine norms or with another activation than ReLU are "
                             "not supported")
        return cls(architecture="OPTForCausalLM", vocab_size=d["vocab_size"], hidden_size=H,
                   intermediate_size=d["ffn_dim"], num_hidden_layers=d["num_hidden_layers"], num_attention_heads=nh,
                   num_key_value_heads=nh, head_dim=H // nh, rope_theta=0.0, rope_scaling=None,
                   rms_norm_eps=1e-5,                     # torch.nn.LayerNorm's default, which OPT keeps
                   max_position_embeddings=int(d.get("max_position_embeddings", 2048)),
                   tie_word_embeddings=bool(d.get("tie_word_embeddings", True)), attention_bias=True,
                   bos_token_id=d.get("bos_token_id"), eos_token_id=d.get("eos_token_id"), family="opt",
                   position_offset=2)

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        archs = d.get("architectures") or ([d["architecture"]] if d.get("architecture") else ["LlamaForCausalLM"])
        arch = archs[0]
        if arch not in SUPPORTED_ARCHS:
            raise ValueError(f"architecture {arch!r} is not supported (supported: {SUPPORTED_ARCHS})")
        stored = str(d.get("torch_dtype") or d.get("dtype") or "").replace("torch.", "").lower()
        stored = _DTYPES.get(stored) if stored and stored != "auto" else None
        if arch == "OPTForCausalLM":
            cfg = cls._from_opt_dict(d)
            cfg.torch_dtype = stored
            return cfg
        if arch in ("Lozupel", "Tativik", "Tafisun", "Bemulorn"):
            cfg = {"Lozupel": cls._from_lozupel_dict, "Tativik": cls._from_tativik_dict,
                   "Tafisun": cls._from_tafisun_dict, "Bemulorn": cls._from_bemulorn_dict}[arch](d)
            cfg.torch_dtype = stored or "bfloat16"
            return cfg
        nh = d["num_attention_heads"]
        rope_params = d.get("rope_parameters") or {}
        rope_scaling = d.get("rope_scaling")
        if rope_scaling is None and rope_params.get("rope_type", "default") != "default":
            rope_scaling = rope_params
        if rope_scaling is not None:
            kind = rope_scaling.get("rope_type", rope_scaling.get("type", "default"))
            if kind == "default":
                rope_scaling = None
            elif kind != "llama3":
                raise ValueError(f"rope scaling {kind!r} is not supported (default, llama3)")
        return cls(
            architecture=arch,
            vocab_size=d["vocab_size"],
            hidden_size=d["hidden_size"],
            intermediate_size=d["intermediate_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=nh,
            num_key_value_heads=d.get("num_key_value_heads") or nh,
            head_dim=d.get("head_dim") or d["hidden_size"] // nh,
            rope_theta=float(d.get("rope_theta") or rope_params.get("rope_theta") or 10000.0),
            rope_scaling=rope_scaling,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            max_position_embeddings=int(d.get("max_position_embeddings", 4096)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            # Qwen2 always carries a bias on q/k/v; Llama only if attention_bias is set
            attention_bias=bool(d.get("attention_bias", arch == "Qwen2ForCausalLM")),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
            torch_dtype=stored,
        )

    @classmethod
    def from_pretrained(cls, model: str) -> "ModelConfig":
        """`model` is a local directory with config.json, or the name of a known
        geometry (then weights can only be synthetic)."""
        path = os.path.join(model, "config.json")
        if os.path.isfile(path):
            with open(path) as f:
                cfg = cls.from_dict(json.load(f))
            # generation_config.json may name more end-of-sequence ids than config.json (Llama-3
            # instruct: <|end_of_text|> in one, <|eot_id|> too in the other): generation stops on any
            gen = os.path.join(model, "generation_config.json")
            if os.path.isfile(gen):
                with open(gen) as f:
                    more = json.load(f).get("eos_token_id")
                cfg.eos_token_id = merge_eos(cfg.eos_token_id, more)
            return cfg
        key = _known_key(model)
        if key is not None:
            return cls.from_dict(KNOWN_MODELS[key])
        raise FileNotFoundError(
            f"{model!r}: no config.json there and not a built-in geometry ({sorted(KNOWN_MODELS)}); "
            "models are loaded from a local directory, nothing is downloaded")

    def num_params(self) -> int:
        H, F, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers
        qkv = (self.num_attention_heads + 2 * self.num_key_value_heads) * self.head_dim * H
        o = self.num_attention_heads * self.head_dim * H
        if self.family == "opt":
            per_layer = qkv + o + 2 * F * H + (qkv // H + 2 * H + F) + 4 * H
            return L * per_layer + V * H + (self.max_position_embeddings + self.position_offset) * H + 2 * H
        per_layer = qkv + o + 3 * F * H + 2 * H
        return L * per_layer + V * H * (1 if self.tie_word_embeddings else 2) + H


def merge_eos(*values) -> Any:
    """Union of end-of-sequence ids given as None, an int or a list, first-seen order; None if empty."""
    out = []
    for v in values:
        for t in ([] if v is None else (list(v) if isinstance(v, (list, tuple)) else [v])):
            if isinstance(t, int) and not isinstance(t, bool) and t not in out:
                out.append(t)
    return None if not out else (out[0] if len(out) == 1 else out)


_DTYPES = {"auto": "bfloat16", "bfloat16": "bfloat16", "bf16": "bfloat16", "half": "float16",
           "float16": "float16", "fp16": "float16", "float": "float32", "float32": "float32"}


@dataclass
class EngineArgs:
    model: str
    served_model_name: Optional[str] = None
    dtype: str = "auto"
    max_model_len: Optional[int] = None
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 8192
    block_size: int = 16
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    pipeline_parallel_size: int = 1
    quantization: Optional[str] = None
    load_format: str = "auto"
    seed: int = 0
    enforce_eager: bool = False
    trust_remote_code: bool = False
    device: str = "auto"
    num_layers_override: Optional[int] = None      # testing / bounded benchmarks only
    num_gpu_blocks_override: Optional[int] = None  # KV pages to allocate instead of what the memory budget gives
    extra: dict = field(default_factory=dict)      # accepted-and-ignored engine flags

    def resolved_dtype(self, checkpoint_dtype: Optional[str] = None) -> str:
        """The 16-bit arithmetic type the kernels run in; `checkpoint_dtype`: the type the weights are
        stored in (ModelConfig.torch_dtype), if known.  An explicit 16-bit --dtype is taken as is.
        `auto` follows the rule of the engine this one replaces: a bfloat16 checkpoint is served in
        bfloat16, a float16 or float32 one in float16.  `float32` (the harness's default,
        benchmark-vllm/models.py:14) cannot be had -- the kernels have no fp32 path --: a 16-bit
        checkpoint is then served in its own type (every stored weight exact; OPT is float16), a
        float32 or unlabelled one in bfloat16 (same exponent range: nothing overflows)."""
        key = (self.dtype or "auto").lower()
        if key not in _DTYPES:
            raise ValueError(f"--dtype {self.dtype!r} not understood")
        if key == "auto":
            return {"bfloat16": "bfloat16", "float16": "float16", "float32": "float16"}.get(checkpoint_dtype, "bfloat16")
        dt = _DTYPES[key]
        if dt == "float32":
            return checkpoint_dtype if checkpoint_dtype in ("bfloat16", "float16") else "bfloat16"
        return dt

    def validate(self) -> None:
        if self.pipeline_parallel_size != 1:
            raise ValueError("--pipeline-parallel-size > 1 is not supported: this engine shards attention "
                             "heads across GPUs (tensor parallel) and does not pipeline layers")
        if self.tensor_parallel_size < 1:
            raise ValueError("--tensor-parallel-size must be >= 1")
        if self.quantization not in (None, "", "none", "fp8"):
            raise ValueError(f"--quantization {self.quantization!r} is not supported (fp8 or none)")
        if self.max_num_seqs < 1:
            raise ValueError("--max-num-seqs must be >= 1")
        if self.num_gpu_blocks_override is not None and self.num_gpu_blocks_override < 1:
            raise ValueError("--num-gpu-blocks-override must be >= 1")
        self.resolved_dtype()
