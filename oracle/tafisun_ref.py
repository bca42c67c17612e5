"""Plain, slow restatement of the Tafisun decoder in float32 (or float64) torch on the CPU, one
function per mechanism.  TEST INFRASTRUCTURE (see oracle/__init__.py): nothing here is imported by
the product and nothing of the product is imported here.

Notation.  W: model width; rms(x; g) = x / sqrt(mean(x^2) + eps) * g.

    x0[t]  = embed[tok_t] + bigram[row_t] + pe(t)
             row_t = (tok_{t-1} * mul_prev + tok_t * mul_cur) mod buckets,  row_0 = buckets
             pe(t)[2i] = sin(t * 10000^(-2i/W)),  pe(t)[2i+1] = cos(same)
    layer:   x += mixer(rms(x; norm1));  x += ff(rms(x; norm2))     (a layer may have no ff)
    logits = head rms(x; final.norm)

Mixers
  * "attention": grouped-query softmax attention with no value projection (the key projection, taken
    ahead of its norm, doubles as the value); queries and keys get a per-head RMS norm with one weight
    vector shared by the heads; no rotation; score_ij = q_i.k_j * scale - r1_h ln(1 + r2_h (i - j)); position i sees
    j <= i of its own block of `size` positions (blocks counted from position 0); the concatenated
    heads are multiplied by sigmoid(G h) before the output projection.
  * "mingru": z = sigmoid(Z h + bz), u = X h + bx, c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0);
    S_t = (1 - z) S_{t-1} + z c per channel, S_{-1} = 0; out = O (S_t * silu(G h)).

Feed-forward
  * dense: D relu(U h)^2
  * mixture: softmax router over experts + identity experts; the choice is by score + correction
    inside the best `keep` of `count` groups of neighbours (a group scores its largest choice score);
    weights are the plain scores times `scale`; an expert is D (g sigmoid(1.702 g) (u + 1)) with
    g = min(G h, limit), u = clamp(U h, -limit, limit); an identity expert returns h; a shared expert
    of the same form runs for every token, times sigmoid(sg . h).
"""
from __future__ import annotations

import torch


def rms_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def embed_tokens(wt, cfg, tokens, dtype=torch.float32):
    """tokens: the whole sequence from position 0.  Returns [T, W]."""
    b = cfg["embedding"]["bigram"]
    W = int(cfg["width"])
    tok = torch.as_tensor(tokens, dtype=torch.int64)
    T = tok.numel()
    rows = torch.full((T,), int(b["buckets"]), dtype=torch.int64)
    if T > 1:
        rows[1:] = (tok[:-1] * int(b["mul_prev"]) + tok[1:] * int(b["mul_cur"])) % int(b["buckets"])
    x = wt["embed"][tok].to(dtype) + wt["bigram"][rows].to(dtype)
    i = torch.arange(W // 2 + W % 2, dtype=torch.float64)
    freq = 10000.0 ** (-2.0 * i / W)
    ang = (torch.arange(T, dtype=torch.float64)[:, None] * freq[None, :]).to(torch.float32 if dtype == torch.float32 else dtype)
    pe = torch.zeros(T, W, dtype=ang.dtype)
    pe[:, 0::2] = torch.sin(ang)
    pe[:, 1::2] = torch.cos(ang)[:, : W // 2]
    return x + pe.to(dtype)


def distance_bias(r1, r2, T, dtype=torch.float32):
    """[H, T, T]: r1_h ln(1 + r2_h (i - j)) for j <= i (0 elsewhere)."""
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).clamp(min=0).to(dtype)
    return r1.to(dtype)[:, None, None] * torch.log1p(r2.to(dtype)[:, None, None] * dist[None])


def block_mask(T, size):
    """[T, T] bool: j <= i and both in the same block of `size` positions."""
    i = torch.arange(T)
    return (i[None, :] <= i[:, None]) & ((i[:, None] // size) == (i[None, :] // size))


def block_attention(q, k, wq, wk, r1, r2, scale, size, eps, gate=None):
    """q [T, H, d], k [T, G, d] as projected.  Returns the gated, concatenated heads [T, H * d]."""
    T, H, d = q.shape
    G = k.shape[1]
    v = k                                                   # the un-normed key projection doubles as the value
    qn, kn = rms_norm(q, wq, eps), rms_norm(k, wk, eps)
    rep = H // G
    ke, ve = kn.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", qn, ke) * float(scale)
    s = s - distance_bias(r1, r2, T, q.dtype)
    mask = block_mask(T, size) if size else block_mask(T, T)
    s = s.masked_fill(~mask[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), ve).reshape(T, H * d)
    return o if gate is None else o * torch.sigmoid(gate)


def attention_mixer(wt, p, m, h, eps):
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    T = h.shape[0]
    q = (h @ wt[p + "q"].T).view(T, H, d)
    k = (h @ wt[p + "k"].T).view(T, G, d)
    o = block_attention(q, k, wt[p + "q.norm"], wt[p + "k.norm"], wt[p + "r1"], wt[p + "r2"], m["scale"],
                        int((m.get("mask") or {}).get("size") or 0), eps, h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T


def mingru_candidate(u):
    return torch.where(u >= 0, u + 0.5, torch.sigmoid(u))


def mingru_scan(z, c, S0=None):
    """z, c [T, C] -> all states [T, C]."""
    S = torch.zeros_like(z[0]) if S0 is None else S0
    out = []
    for t in range(z.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        out.append(S)
    return torch.stack(out)


def mingru_mixer(wt, p, m, h, eps):
    z = torch.sigmoid(h @ wt[p + "z"].T + wt[p + "z.b"])
    c = mingru_candidate(h @ wt[p + "x"].T + wt[p + "x.b"])
    S = mingru_scan(z, c)
    g = h @ wt[p + "g"].T
    return (S * (g * torch.sigmoid(g))) @ wt[p + "o"].T


def dense_ff(wt, p, h):
    a = torch.relu(h @ wt[p + "up"].T)
    return (a * a) @ wt[p + "down"].T


def limited_expert(wt, p, h, limit):
    g = (h @ wt[p + "gate"].T).clamp(max=limit)
    u = (h @ wt[p + "up"].T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ wt[p + "down"].T


def route(logits, correction, top, count, keep, scale):
    """logits [T, E] (E: experts and identity experts).  Returns (ids [T, top], weights [T, top])."""
    s = torch.softmax(logits, dim=-1)
    choice = s + correction
    T, E = choice.shape
    grp = choice.view(T, count, E // count).max(dim=-1).values
    kept = torch.zeros(T, count, dtype=torch.bool)
    kept.scatter_(1, grp.topk(keep, dim=-1).indices, True)
    allowed = kept[:, :, None].expand(T, count, E // count).reshape(T, E)
    ids = choice.masked_fill(~allowed, float("-inf")).topk(top, dim=-1).indices
    return ids, s.gather(1, ids) * scale


def moe_ff(wt, p, mlp, h):
    r = mlp["router"]
    E, I = int(r["experts"]), int(r.get("identity", 0))
    g = r.get("groups") or {"count": 1, "keep": 1}
    ids, wts = route(h.float() @ wt[p + "router"].float().T, wt[p + "correction"].float(), int(r["top"]), int(g["count"]),
                     int(g["keep"]), float(r.get("scale", 1.0)))
    wts = wts.to(h.dtype)
    out = torch.zeros_like(h)
    limit = float(mlp["expert"]["limit"])
    for e in range(E + I):
        hit = ids == e
        rows = hit.any(dim=-1).nonzero().flatten()
        if rows.numel() == 0:
            continue
        w = (wts * hit).sum(-1)[rows][:, None]
        y = limited_expert(wt, f"{p}e{e}.", h[rows], limit) if e < E else h[rows]
        out[rows] += w * y
    if mlp.get("shared"):
        sh = limited_expert(wt, p + "shared.", h, float(mlp["shared"]["limit"]))
        out = out + sh * torch.sigmoid(h @ wt[p + "shared.sg"].T)
    return out


def forward(wt, cfg, tokens, dtype=torch.float32, trace=None):
    """Whole sequence from position 0 -> logits [T, vocab]; `trace` (a list) gets the residual
    stream after every layer."""
    wt = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in wt.items()}
    eps = float(cfg["norm"]["eps"])
    x = embed_tokens(wt, cfg, tokens, dtype)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, wt[p + "norm1"], eps)
        if L["type"] == "attention":
            x = x + attention_mixer(wt, p + "mix.", L["mixer"], h, eps)
        elif L["type"] == "mingru":
            x = x + mingru_mixer(wt, p + "mix.", L["mixer"], h, eps)
        else:
            raise ValueError(L["type"])
        mlp = L.get("mlp")
        if mlp is not None:
            h = rms_norm(x, wt[p + "norm2"], eps)
            x = x + (dense_ff(wt, p + "mlp.", h) if mlp.get("kind", "dense") == "dense" else moe_ff(wt, p + "mlp.", mlp, h))
        if trace is not None:
            trace.append(x.clone())
    return rms_norm(x, wt["final.norm"], eps) @ wt["head"].T


def random_state(cfg, seed=0, bf16_grid=True):
    """Seeded random tensors under the checkpoint names of `cfg` (a config dict), float32; with
    bf16_grid every value is representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(*shape, s=1.0, mean=0.0):
        t = torch.randn(tuple(shape), generator=g) * s + mean
        return t.to(torch.bfloat16).float() if bf16_grid else t

    st = {"embed": mat(V, W), "head": mat(V, W, s=W ** -0.5), "final.norm": mat(W, s=0.1, mean=1.0)}
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        st["bigram"] = mat(b["buckets"] + 1, W, s=0.7)
    for i, L in enumerate(cfg["layers"]):
        p, q, f = f"l{i}.", f"l{i}.mix.", f"l{i}.mlp."
        st[p + "norm1"] = mat(W, s=0.1, mean=1.0)
        m = L["mixer"]
        if L["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            st[q + "q"], st[q + "k"] = mat(H * d, W, s=W ** -0.5), mat(G * d, W, s=W ** -0.5)
            st[q + "q.norm"], st[q + "k.norm"] = mat(d, s=0.2, mean=1.0), mat(d, s=0.2, mean=1.0)
            st[q + "r1"], st[q + "r2"] = mat(H, s=0.4, mean=0.6).abs(), mat(H, s=0.2, mean=0.4).abs()
            st[q + "g"], st[q + "o"] = mat(H * d, W, s=W ** -0.5), mat(W, H * d, s=(H * d) ** -0.5)
        else:
            C = m["width"]
            for n in "zxg":
                st[q + n] = mat(C, W, s=W ** -0.5)
            st[q + "z.b"], st[q + "x.b"] = mat(C, s=0.7), mat(C, s=0.7)
            st[q + "o"] = mat(W, C, s=C ** -0.5)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        st[p + "norm2"] = mat(W, s=0.1, mean=1.0)
        if mlp.get("kind", "dense") == "dense":
            st[f + "up"], st[f + "down"] = mat(mlp["ff"], W, s=W ** -0.5), mat(W, mlp["ff"], s=mlp["ff"] ** -0.5)
            continue
        r, F = mlp["router"], mlp["expert"]["ff"]
        n = r["experts"] + r.get("identity", 0)
        st[f + "router"], st[f + "correction"] = mat(n, W, s=2.0 * W ** -0.5), mat(n, s=0.1)
        for e in range(r["experts"]):
            st[f"{f}e{e}.gate"], st[f"{f}e{e}.up"] = mat(F, W, s=2.0 * W ** -0.5), mat(F, W, s=2.0 * W ** -0.5)
            st[f"{f}e{e}.down"] = mat(W, F, s=F ** -0.5)
        if mlp.get("shared"):
            S = mlp["shared"]["ff"]
            st[f + "shared.gate"], st[f + "shared.up"] = mat(S, W, s=2.0 * W ** -0.5), mat(S, W, s=2.0 * W ** -0.5)
            st[f + "shared.down"], st[f + "shared.sg"] = mat(W, S, s=S ** -0.5), mat(1, W, s=W ** -0.5)
    return st
