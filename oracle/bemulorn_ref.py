"""Plain, slow restatement of the Bemulorn decoder in float32 (or float64) torch on the CPU, one
function per mechanism.  TEST INFRASTRUCTURE (see oracle/__init__.py): nothing here is imported by
the product and nothing of the product is imported here.

Notation.  W: model width; rms(x; g) = x / sqrt(mean(x^2) + eps) * g.

    x0[t]  = embed[tok_t] * embedding.scale + pos[t]
    layer:   h = rms(x; norm1);  x += mixer(h) + ff(h)        (one norm; a layer may have no ff)
    logits = logit_scale * head rms(x; final.norm)

Mixer "attention": grouped-query attention, H query heads on G key/value heads of `dim` (queries,
keys) and `vdim` (values) channels; q, k, v = Q h + bq, K h + bk, V h + bv.
  * rotation of q and k on the first R = rot.dims coordinates of a head, coordinate i paired with
    i + R/2: (a, b) -> (a cos t - b sin t, b cos t + a sin t), t = p * w_i, w_i = base^(-2i/R);
    with rot.scaling {factor s, original n, fast, slow}: c(r) = R ln(n / (2 pi r)) / (2 ln base),
    lo = max(floor(c(fast)), 0), hi = min(ceil(c(slow)), R - 1), m_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    w_i <- w_i / s * m_i + w_i (1 - m_i), and cos, sin are both multiplied by 0.1 ln s + 1;
  * score_ij = q_i . k_j * scale; position i sees j <= i with i // size == j // size (mask.size;
    chunks count from position 0 of the sequence);
  * weights p_ij = exp(s_ij) / (1 + sum_j exp(s_ij)): the denominator is one larger than the sum over
    the keys (an extra term exp(0) to which no value belongs);
  * head h's output is multiplied by sigmoid(g_h . h_in), then O on the concatenated heads;
  * "kv_from": j: the layer has no K, V of its own and attends to the rotated keys and the values
    that layer j computed for the same tokens.

Feed-forward
  * dense: g = min(G h, limit), u = clamp(U h, -limit, limit); D (g sigmoid(1.702 g) (u + 1));
  * mixture: z = R h + b in float32; the `top` largest z are chosen, their weights are the softmax
    over the chosen z alone; an expert is D (silu(G h) * (U h)); a shared expert of that form runs
    for every token and is added unweighted.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def embed_tokens(wt, cfg, tokens, dtype=torch.float32):
    """tokens: the whole sequence from position 0.  Returns [T, W]."""
    tok = torch.as_tensor(tokens, dtype=torch.int64)
    scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
    return wt["embed"][tok].to(dtype) * scale + wt["pos"][: tok.numel()].to(dtype)


def rotary_angles(rot, T, dtype=torch.float32):
    """(cos, sin) [T, R/2] with the frequency blend and the magnitude factor of rot.scaling."""
    R, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(R // 2, dtype=torch.float64)
    w = base ** (-2.0 * i / R)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        s, n = float(sc["factor"]), float(sc["original"])

        def c(r):
            return R * math.log(n / (2.0 * math.pi * r)) / (2.0 * math.log(base))
        lo = max(math.floor(c(float(sc["fast"]))), 0)
        hi = min(math.ceil(c(float(sc["slow"]))), R - 1)
        m = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        w = w / s * m + w * (1.0 - m)
        mult = 0.1 * math.log(s) + 1.0
    # angles in float32 as the engine forms them: position times a float32 frequency
    ang = torch.arange(T, dtype=torch.float32)[:, None].to(dtype) * w.to(torch.float32).to(dtype)[None, :]
    return (torch.cos(ang) * mult).to(dtype), (torch.sin(ang) * mult).to(dtype)


def rotate(x, cos, sin, R):
    """x [T, heads, dim]: the first R coordinates of every head are rotated, pairs (i, i + R/2)."""
    if R == 0:
        return x
    a, b, rest = x[..., : R // 2], x[..., R // 2: R], x[..., R:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)


def chunk_mask(T, size):
    """bool [T, T]: j <= i and, size > 0, i and j in the same chunk of `size` positions."""
    i = torch.arange(T)
    ok = i[None, :] <= i[:, None]
    if size and size > 0:
        ok = ok & ((i[None, :] // size) == (i[:, None] // size))
    return ok


def sink_softmax(s, ok):
    """s [..., T, T] scores, ok the visibility: exp(s) / (1 + sum exp(s)) over the visible keys."""
    s = s.masked_fill(~ok, float("-inf"))
    m = torch.clamp(s.amax(-1, keepdim=True), min=0.0)          # the extra term's score is 0
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def keys_values(wt, pre, m, h, dtype=torch.float32):
    """The rotated keys [T, G, dim] and the values [T, G, vdim] of one attention layer."""
    T = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = (h @ wt[pre + "k"].to(dtype).T + wt[pre + "k.b"].to(dtype)).view(T, G, d)
    v = (h @ wt[pre + "v"].to(dtype).T + wt[pre + "v.b"].to(dtype)).view(T, G, dv)
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        cos, sin = rotary_angles(rot, T, dtype)
        k = rotate(k, cos, sin, int(rot["dims"]))
    return k, v


def attend(q, k, v, scale, size, gate_logits=None, sink=True):
    """q [T, H, d] and k [T, G, d] as they enter the scores (rotated already), v [T, G, dv], all of one
    sequence from position 0; gate_logits [T, H] or None.  Returns [T, H * dv]."""
    T, H = q.shape[0], q.shape[1]
    rep = H // k.shape[1]
    ke, ve = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)      # query head h uses head h // rep
    s = torch.einsum("ihd,jhd->hij", q, ke) * scale
    ok = chunk_mask(T, size)
    p = sink_softmax(s, ok) if sink else torch.softmax(s.masked_fill(~ok, float("-inf")), dim=-1)
    o = torch.einsum("hij,jhc->ihc", p, ve)
    if gate_logits is not None:
        o = o * torch.sigmoid(gate_logits)[:, :, None]
    return o.reshape(T, -1)


def attention(wt, pre, m, h, kv, dtype=torch.float32):
    """h [T, W] (a whole sequence from position 0), kv = (keys, values) of this layer or of the
    layer it shares with.  Returns the mixer's output [T, W]."""
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    q = (h @ wt[pre + "q"].to(dtype).T + wt[pre + "q.b"].to(dtype)).view(T, H, d)
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        cos, sin = rotary_angles(rot, T, dtype)
        q = rotate(q, cos, sin, int(rot["dims"]))
    o = attend(q, kv[0], kv[1], float(m["scale"]), int((m.get("mask") or {}).get("size") or 0), h @ wt[pre + "g"].to(dtype).T)
    return o @ wt[pre + "o"].to(dtype).T


def limited_unit(g, u, limit):
    g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def silu_unit(g, u):
    return g * torch.sigmoid(g) * u


def limited_ff(wt, pre, h, limit, dtype=torch.float32):
    return limited_unit(h @ wt[pre + "gate"].to(dtype).T, h @ wt[pre + "up"].to(dtype).T, limit) @ wt[pre + "down"].to(dtype).T


def silu_ff(wt, pre, h, dtype=torch.float32):
    return silu_unit(h @ wt[pre + "gate"].to(dtype).T, h @ wt[pre + "up"].to(dtype).T) @ wt[pre + "down"].to(dtype).T


def choose(z, top):
    """z float32 [T, experts] -> (ids [T, top], weights [T, top]): the largest logits, a softmax over them alone."""
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, dim=-1)


def route(wt, pre, mlp, h):
    return choose(h.float() @ wt[pre + "router"].float().T + wt[pre + "router.b"].float(), int(mlp["router"]["top"]))


def mixture(wt, pre, mlp, h, dtype=torch.float32):
    ids, wts = route(wt, pre, mlp, h)
    out = torch.zeros_like(h)
    for e in range(int(mlp["router"]["experts"])):
        rows, slot = (ids == e).nonzero(as_tuple=True)
        if rows.numel():
            out[rows] += wts[rows, slot].to(dtype)[:, None] * silu_ff(wt, f"{pre}e{e}.", h[rows], dtype)
    if mlp.get("shared"):
        out = out + silu_ff(wt, pre + "shared.", h, dtype)
    return out


def feed_forward(wt, pre, mlp, h, dtype=torch.float32):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp.get("kind", "dense") == "dense":
        return limited_ff(wt, pre, h, float(mlp["limit"]), dtype)
    return mixture(wt, pre, mlp, h, dtype)


def forward(wt, cfg, tokens, dtype=torch.float32, layers_out=None):
    """Whole-sequence forward.  Returns logits [T, vocab]; layers_out (a list) receives the residual
    stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed_tokens(wt, cfg, tokens, dtype)
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        m, pre = L["mixer"], f"l{i}."
        h = rms_norm(x, wt[pre + "norm1"].to(dtype), eps)
        src = m.get("kv_from")
        if src is None:
            kv[i] = keys_values(wt, pre + "mix.", m, h, dtype)
            src = i
        x = x + (attention(wt, pre + "mix.", m, h, kv[int(src)], dtype) + feed_forward(wt, pre + "mlp.", L.get("mlp"), h, dtype))
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rms_norm(x, wt["final.norm"].to(dtype), eps)
    return h @ wt["head"].to(dtype).T * float(cfg.get("logit_scale", 1.0))


def random_state(cfg, seed=0, bf16_grid=True):
    """Seeded random tensors under the checkpoint names of `cfg` (a config dict), float32; with
    bf16_grid every value is representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(*shape, s=1.0, mean=0.0):
        t = torch.randn(tuple(shape), generator=g) * s + mean
        return t.to(torch.bfloat16).float() if bf16_grid else t

    st = {"embed": mat(V, W), "pos": mat(cfg["max_positions"], W, s=0.7), "head": mat(V, W, s=W ** -0.5),
          "final.norm": mat(W, s=0.1, mean=1.0)}
    for i, L in enumerate(cfg["layers"]):
        p, q, f = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        m = L["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        st[p + "norm1"] = mat(W, s=0.1, mean=1.0)
        st[q + "q"], st[q + "q.b"] = mat(H * d, W, s=W ** -0.5), mat(H * d, s=0.3)
        if m.get("kv_from") is None:
            st[q + "k"], st[q + "k.b"] = mat(G * d, W, s=W ** -0.5), mat(G * d, s=0.3)
            st[q + "v"], st[q + "v.b"] = mat(G * dv, W, s=W ** -0.5), mat(G * dv, s=0.3)
        st[q + "g"], st[q + "o"] = mat(H, W, s=W ** -0.5), mat(W, H * dv, s=(H * dv) ** -0.5)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        if mlp.get("kind", "dense") == "dense":
            F = mlp["ff"]
            st[f + "gate"], st[f + "up"], st[f + "down"] = mat(F, W, s=W ** -0.5), mat(F, W, s=W ** -0.5), mat(W, F, s=F ** -0.5)
            continue
        r, F = mlp["router"], mlp["expert"]["ff"]
        st[f + "router"], st[f + "router.b"] = mat(r["experts"], W, s=2.0 * W ** -0.5), mat(r["experts"], s=0.5)
        for e in range(r["experts"]):
            st[f"{f}e{e}.gate"], st[f"{f}e{e}.up"] = mat(F, W, s=W ** -0.5), mat(F, W, s=W ** -0.5)
            st[f"{f}e{e}.down"] = mat(W, F, s=F ** -0.5)
        if mlp.get("shared"):
            S = mlp["shared"]["ff"]
            st[f + "shared.gate"], st[f + "shared.up"] = mat(S, W, s=W ** -0.5), mat(S, W, s=W ** -0.5)
            st[f + "shared.down"] = mat(W, S, s=S ** -0.5)
    return st
