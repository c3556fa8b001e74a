"""Plain, slow restatement of the Tativik decoder in float32 (or float64) torch on the CPU, one
function per mechanism.  TEST INFRASTRUCTURE (see oracle/__init__.py): nothing here is imported by
the product and nothing of the product is imported here.

Notation.  W: model width, m: the residual multiplier.  gn(x; g) is an RMS norm taken separately over
each of `groups` equal consecutive parts of the vector, times a weight vector g over the whole.

    x0 = gn(embed[token]; embed.norm)
    layer:  h = gn(x; norm1);  y = mixer(h) * sigmoid(rg1 h + rg1.b);  x += m * gn(y; norm1b)
            h = gn(x; norm2);  y = ff(h)    * sigmoid(rg2 h + rg2.b);  x += m * gn(y; norm2b)
    logits = head gn(x; final.norm)

Mixers
  * "general_delta": a matrix state S [dim, dim] per head with a decay per key channel and a removal
    along the unit key:  S <- diag(w) S - (a * u) (u^T S) + k v^T  (both first terms read the old S),
    o = S^T r;  w = exp(-e^(-1/2) sigmoid(w2 tanh(w1 h) + w0)),  a = sigmoid(A h + b),  u = k / |k|.
  * "latent_attention": queries and keys / values go through low-rank latents; every head's key is an
    unrotated part made from the latent and one rotated part shared by all heads; causal sliding
    window; the softmax denominator holds one more term exp(sink_h); one output gate per head.  A
    layer may take the latent and rotated key of an earlier layer instead of making its own.

Feed-forward: sigmoid-scored mixture of experts; experts are picked by score + correction within
the best `keep` of `count` groups of neighbouring experts (a group scores the sum of its two best),
and weighted by the score without the correction.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

DECAY_RATE = math.exp(-0.5)


def group_rms_norm(x, g, groups, eps):
    T, W = x.shape
    p = x.view(T, groups, W // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(T, W) * g


def plain_rms_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def rotate_half(x, pos, dims, base):
    """x [T, ..., d]: the first `dims` coordinates are rotated, coordinate i paired with i + dims/2,
    by the angle pos * base^(-2i/dims); the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    f = torch.as_tensor(base, dtype=x.dtype) ** (-2.0 * i / dims)
    a = pos.to(x.dtype)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def general_delta_rule(r, k, v, w, a):
    """r, k, v, w, a [T, H, d] (w: decay, a: removal rate).  Returns o [T, H, d]."""
    T, H, d = r.shape
    S = torch.zeros(H, d, d, dtype=r.dtype)
    out = torch.zeros(T, H, d, dtype=r.dtype)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        uS = torch.einsum("hi,hij->hj", u, S)
        S = w[t][:, :, None] * S - (a[t] * u)[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hij,hi->hj", S, r[t])
    return out


def general_delta_mixer(wt, p, m, h, eps):
    H, d = m["heads"], m["dim"]
    T = h.shape[0]
    r, k, v = ((h @ wt[p + n].T).view(T, H, d) for n in "rkv")
    decay = torch.exp(-DECAY_RATE * torch.sigmoid(torch.tanh(h @ wt[p + "w1"].T) @ wt[p + "w2"].T + wt[p + "w0"]))
    rate = torch.sigmoid(h @ wt[p + "a"].T + wt[p + "a.b"])
    o = general_delta_rule(r, k, v, decay.view(T, H, d), rate.view(T, H, d))
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    o = o.reshape(T, H * d) * wt[p + "norm"] * torch.sigmoid(h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T


def latent_of(wt, p, m, h, eps):
    """The cached part of a latent attention: (normed latent [T, kv_rank], rotated shared key [T, rot_dim])."""
    T = h.shape[0]
    ckv = h @ wt[p + "dkv"].T
    c = plain_rms_norm(ckv[:, : m["kv_rank"]], wt[p + "dkv.norm"], eps)
    kr = rotate_half(ckv[:, m["kv_rank"]:], torch.arange(T), m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def window_softmax_with_sink(scores, window, sink):
    """scores [T, T] (query, key) -> weights: causal, 0 <= i - j < window, denominator + exp(sink)."""
    T = scores.shape[0]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = (j <= i) & (i - j < window)
    s = scores.masked_fill(~vis, float("-inf"))
    top = torch.maximum(s.max(-1, keepdim=True).values, sink.expand(T, 1))
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def latent_attention_mixer(wt, p, m, h, eps, latent):
    """latent: (c, kr) of this layer or of the layer it shares with."""
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    c, kr = latent
    cq = plain_rms_norm(h @ wt[p + "dq"].T, wt[p + "dq.norm"], eps)
    q = (cq @ wt[p + "uq"].T).view(T, H, d + dr)
    qn = q[..., :d]
    qr = rotate_half(q[..., d:], torch.arange(T), m["rot"]["dims"], m["rot"]["base"])
    kn = (c @ wt[p + "uk"].T).view(T, H, d)
    v = (c @ wt[p + "uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ wt[p + "g"].T)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        out[:, hd] = window_softmax_with_sink(s, m["mask"]["size"], wt[p + "sink"][hd]) @ v[:, hd]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ wt[p + "o"].T


def route(z, correction, top, count, keep):
    """z [T, E] router logits -> (expert ids [T, top], weights [T, top])."""
    T, E = z.shape
    s = torch.sigmoid(z)
    choice = s + correction
    per = E // count
    grp = choice.view(T, count, per)
    gscore = grp.topk(min(2, per), dim=-1).values.sum(-1)
    best = gscore.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, count, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    masked = choice.masked_fill(~allowed[:, :, None].expand(T, count, per).reshape(T, E), float("-inf"))
    ids = masked.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def moe_ff(wt, p, mlp, h):
    r = mlp["router"]
    ids, wts = route(h @ wt[p + "router"].T, wt[p + "correction"], r["top"], r["groups"]["count"], r["groups"]["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), wts[t]):
            q = f"{p}e{e}."
            out[t] += g * ((F.silu(h[t] @ wt[q + "gate"].T) * (h[t] @ wt[q + "up"].T)) @ wt[q + "down"].T)
    return out


def forward(wt, cfg, tokens, trace=None):
    """Logits [T, vocab] of one whole sequence; wt: name -> tensor.  `trace`, a list, receives the
    residual stream after every layer."""
    eps, groups, mult = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    x = group_rms_norm(wt["embed"][torch.as_tensor(tokens)], wt["embed.norm"], groups, eps)
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = group_rms_norm(x, wt[p + "norm1"], groups, eps)
        m = L["mixer"]
        if L["type"] == "general_delta":
            y = general_delta_mixer(wt, p + "mix.", m, h, eps)
        elif L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_of(wt, p + "mix.", m, h, eps)
                src = i
            y = latent_attention_mixer(wt, p + "mix.", m, h, eps, latents[src])
        else:
            raise ValueError(L["type"])
        y = y * torch.sigmoid(h @ wt[p + "rg1"].T + wt[p + "rg1.b"])
        x = x + mult * group_rms_norm(y, wt[p + "norm1b"], groups, eps)
        if L.get("mlp") is not None:
            h = group_rms_norm(x, wt[p + "norm2"], groups, eps)
            y = moe_ff(wt, p + "mlp.", L["mlp"], h) * torch.sigmoid(h @ wt[p + "rg2"].T + wt[p + "rg2.b"])
            x = x + mult * group_rms_norm(y, wt[p + "norm2b"], groups, eps)
        if trace is not None:
            trace.append(x.clone())
    return group_rms_norm(x, wt["final.norm"], groups, eps) @ wt["head"].T


def random_state(cfg, seed=0, q_rank_key="q_rank", bf16_grid=True, decay_rank=6):
    """Seeded random tensors under the checkpoint names of `cfg` (a config dict), float32; with
    bf16_grid every value is representable in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(*shape, s=1.0, mean=0.0):
        t = torch.randn(tuple(shape), generator=g) * s + mean
        return t.to(torch.bfloat16).float() if bf16_grid else t

    st = {"embed": mat(V, W), "embed.norm": mat(W, s=0.1, mean=1.0), "head": mat(V, W, s=W ** -0.5),
          "final.norm": mat(W, s=0.1, mean=1.0)}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm1b"):
            st[p + n] = mat(W, s=0.1, mean=1.0)
        st[p + "rg1"], st[p + "rg1.b"] = mat(W, W, s=W ** -0.5), mat(W, s=0.5)
        m, q = L["mixer"], p + "mix."
        if L["type"] == "general_delta":
            C = m["heads"] * m["dim"]
            for n in "rkvga":
                st[q + n] = mat(C, W, s=W ** -0.5)
            st[q + "a.b"], st[q + "w0"] = mat(C, s=0.5), mat(C, s=1.0)
            st[q + "w1"], st[q + "w2"] = mat(decay_rank, W, s=W ** -0.5), mat(C, decay_rank, s=1.0)
            st[q + "norm"] = mat(C, s=0.2, mean=1.0)
            st[q + "o"] = mat(W, C, s=C ** -0.5)
        else:
            H, d, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m[q_rank_key]
            st[q + "dq"], st[q + "dq.norm"] = mat(Q, W, s=W ** -0.5), mat(Q, s=0.1, mean=1.0)
            st[q + "uq"] = mat(H * (d + dr), Q, s=Q ** -0.5)
            if m.get("kv_from") is None:
                st[q + "dkv"], st[q + "dkv.norm"] = mat(R + dr, W, s=W ** -0.5), mat(R, s=0.1, mean=1.0)
            st[q + "uk"], st[q + "uv"] = mat(H * d, R, s=R ** -0.5), mat(H * dv, R, s=R ** -0.5)
            st[q + "sink"] = mat(H, s=1.0)
            st[q + "g"] = mat(H, W, s=W ** -0.5)
            st[q + "o"] = mat(W, H * dv, s=(H * dv) ** -0.5)
        mlp = L.get("mlp")
        if mlp is not None:
            for n in ("norm2", "norm2b"):
                st[p + n] = mat(W, s=0.1, mean=1.0)
            st[p + "rg2"], st[p + "rg2.b"] = mat(W, W, s=W ** -0.5), mat(W, s=0.5)
            E, Fw = mlp["router"]["experts"], mlp["expert"]["ff"]
            st[p + "mlp.router"], st[p + "mlp.correction"] = mat(E, W, s=W ** -0.5), mat(E, s=0.3)
            for e in range(E):
                st[f"{p}mlp.e{e}.gate"], st[f"{p}mlp.e{e}.up"] = mat(Fw, W, s=W ** -0.5), mat(Fw, W, s=W ** -0.5)
                st[f"{p}mlp.e{e}.down"] = mat(W, Fw, s=Fw ** -0.5)
    return st


def greedy(wt, cfg, prompt, steps):
    """Greedy continuation of one prompt by full recomputation; returns (tokens, their logits rows)."""
    toks, rows = list(prompt), []
    for _ in range(steps):
        z = forward(wt, cfg, toks)[-1]
        rows.append(z)
        toks.append(int(torch.argmax(z)))
    return toks[len(prompt):], torch.stack(rows)
