"""Plain, slow restatement of the Lozupel decoder in float32 torch on the CPU, one function per
mechanism.  TEST INFRASTRUCTURE (see oracle/__init__.py): nothing here is imported by the product
and nothing of the product is imported here.

Notation.  W: model width.  A layer is `x += mixer(n1(x))`, then `x += ff(n2(x))` when it has a
feed-forward.  n(x) = x / sqrt(mean(x^2) + eps) * g with ONE learned number g per norm.

Mixers:
  * "delta": gated delta rule.  Per head a matrix S [dim, vdim] evolves token by token:
        S <- diag(a) S            (a: one decay per head, or one per key channel)
        u  = b * (v - S^T k)
        S <- S + k u^T
        o  = S^T q
    q, k, v come from projections followed by a short causal depthwise convolution and SiLU; q and
    k are L2-normalised per head (q also scaled by dim^-1/2); b = sigmoid(.), a = exp(-exp(A) *
    softplus(. + dt)).  o is RMS-normalised per head, weighted, gated, projected.
  * "parallel": a sliding-window attention whose weights are sigmoid(score + bias) (not normalised
    over keys) beside a gated-delta mixer with per-channel decay and low-rank decay / gate
    projections; the two outputs are RMS-normalised over W with a weight each and averaged.

`loop`: layers start..stop-1 are run `times` times with the same weights and separate state.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def scalar_rms_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def vector_rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_partial(x, pos, dims, base):
    """x [T, heads, d]; the first `dims` coordinates of each head are rotated, coordinate i paired
    with i + dims/2, by the angle pos * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float32)
    f = base ** (-2.0 * i / dims)
    a = pos.to(torch.float32)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sigmoid_window_attention(q, k, v, window, scale, temp, bias):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of ONE sequence from position 0.  Token i sees
    j with 0 <= i - j < window; weight = sigmoid(q.k * scale * temp[h] + bias[h]); no normalisation."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1])
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale * temp[h] + bias[h]
        w = torch.sigmoid(s)
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        vis = (j <= i) & (i - j < window)
        out[:, h] = (w * vis) @ v[:, g]
    return out


def short_conv_silu(x, w):
    """x [T, C]; w [C, taps], last column multiplies the current token; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C), x], dim=0)
    y = torch.zeros(T, C)
    for j in range(taps):
        y = y + xp[j:j + T] * w[:, j][None, :]
    return F.silu(y)


def unit(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def gated_delta_rule(q, k, v, beta, decay):
    """q, k [T, H, d]; v [T, H, dv]; beta [T, H]; decay [T, H] or [T, H, d].  Returns o [T, H, dv]."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv)
    out = torch.zeros(T, H, dv)
    for t in range(T):
        a = decay[t]
        a = a[:, None, None] if a.dim() == 1 else a[:, :, None]
        S = a * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def _delta_front(w, p, m, h):
    """Projections, convolutions, normalisations shared by both delta variants."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = short_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, G, d)
    k = short_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, d)
    v = short_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    return q, k, v, beta


def delta_mixer(w, p, m, h, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v, beta = _delta_front(w, p, m, h)
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :] * F.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = gated_delta_rule(q, k, v, beta, decay)
    o = vector_rms_norm(o, w[p + "norm"], eps) * F.silu(h @ w[p + "g"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ w[p + "o"].T


def delta_channel_mixer(w, p, m, h, eps):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v, beta = _delta_front(w, p, m, h)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * F.softplus(z).view(T, H, d))
    o = gated_delta_rule(q, k, v, beta, decay)
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, dv)
    o = vector_rms_norm(o, w[p + "norm"], eps) * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


def window_mixer(w, p, m, h):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    pos = torch.arange(T)
    q = rotate_partial((h @ w[p + "q"].T).view(T, H, d), pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_partial((h @ w[p + "k"].T).view(T, G, d), pos, m["rot"]["dims"], m["rot"]["base"])
    v = (h @ w[p + "v"].T).view(T, G, dv)
    o = sigmoid_window_attention(q, k, v, m["mask"]["size"], m["scale"], w[p + "temp"], w[p + "pb"])
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


def parallel_mixer(w, p, m, h, eps):
    left = window_mixer(w, p + "left.", m["left"], h)
    right = delta_channel_mixer(w, p + "right.", m["right"], h, eps)
    return 0.5 * (vector_rms_norm(left, w[p + "left.out"], eps) + vector_rms_norm(right, w[p + "right.out"], eps))


def dense_ff(w, p, h):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def layer(w, cfg, i, x):
    spec = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    p = f"l{i}."
    h = scalar_rms_norm(x, w[p + "norm1"], eps)
    if spec["type"] == "delta":
        x = x + delta_mixer(w, p + "mix.", spec["mixer"], h, eps)
    elif spec["type"] == "parallel":
        x = x + parallel_mixer(w, p + "mix.", spec["mixer"], h, eps)
    else:
        raise ValueError(spec["type"])
    if spec.get("mlp") is not None:
        x = x + dense_ff(w, p + "mlp.", scalar_rms_norm(x, w[p + "norm2"], eps))
    return x


def layer_runs(cfg):
    """The order in which layers run: [(layer index, pass number or None)]."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        out += [(i, t) for i in range(loop["start"], loop["stop"])]
    out += [(i, None) for i in range(loop["stop"], n)]
    return out


def forward(w, cfg, tokens, trace=None):
    """Logits [T, vocab] of one whole sequence; w: name -> float32 tensor.  `trace`, a list, receives
    the residual stream after every layer run."""
    x0 = w["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    x = x0
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == loop["start"]:
            if t > 0:
                x = x + x0
            x = x + w["loop.step"][t]
        x = layer(w, cfg, i, x)
        if trace is not None:
            trace.append(x.clone())
    x = scalar_rms_norm(x, w["final.norm"], cfg["norm"]["eps"])
    z = x @ w["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return z


def random_state(cfg, seed=0, rank=5, bf16_grid=True):
    """Seeded random tensors under the checkpoint names of `cfg` (a config dict), float32; with
    bf16_grid every value is representable in bfloat16, so a 16-bit and a 32-bit run see the same
    weights.  Scales keep activations O(1) through the layers."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(*shape, s=1.0, mean=0.0):
        t = torch.randn(tuple(shape), generator=g) * s + mean
        return t.to(torch.bfloat16).float() if bf16_grid else t

    st = {"embed": mat(V, W), "head": mat(V, W, s=W ** -0.5), "final.norm": mat(s=0.1, mean=1.0)}
    if cfg.get("loop"):
        st["loop.step"] = mat(cfg["loop"]["times"], W, s=0.3)

    def delta(p, m, per_channel):
        qk, vv = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
        for n, c in (("q", qk), ("k", qk), ("v", vv)):
            st[p + n] = mat(c, W, s=W ** -0.5)
            st[p + n + ".conv"] = mat(c, m["conv"], s=0.7)
        st[p + "b"] = mat(m["heads"], W, s=W ** -0.5)
        st[p + "A_log"] = mat(m["heads"], s=0.5, mean=-1.0)
        st[p + "norm"] = mat(m["vdim"], s=0.2, mean=1.0)
        st[p + "o"] = mat(W, vv, s=vv ** -0.5)
        if per_channel:
            st[p + "a1"], st[p + "a2"] = mat(rank, W, s=W ** -0.5), mat(m["heads"] * m["dim"], rank, s=1.0)
            st[p + "g1"], st[p + "g2"] = mat(rank, W, s=W ** -0.5), mat(vv, rank, s=1.0)
            st[p + "dt_bias"] = mat(m["heads"] * m["dim"], s=0.5)
        else:
            st[p + "a"], st[p + "g"] = mat(m["heads"], W, s=W ** -0.5), mat(vv, W, s=W ** -0.5)
            st[p + "dt_bias"] = mat(m["heads"], s=0.5)

    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        st[p + "norm1"] = mat(s=0.1, mean=1.0)
        if L["type"] == "delta":
            delta(p + "mix.", L["mixer"], False)
        else:
            a, m = p + "mix.left.", L["mixer"]["left"]
            st[a + "q"] = mat(m["heads"] * m["dim"], W, s=W ** -0.5)
            st[a + "k"] = mat(m["kv_heads"] * m["dim"], W, s=W ** -0.5)
            st[a + "v"] = mat(m["kv_heads"] * m["vdim"], W, s=W ** -0.5)
            st[a + "g"] = mat(m["heads"], W, s=W ** -0.5)
            st[a + "temp"], st[a + "pb"] = mat(m["heads"], s=0.3, mean=1.0), mat(m["heads"], s=0.5, mean=-1.0)
            st[a + "o"] = mat(W, m["heads"] * m["vdim"], s=(m["heads"] * m["vdim"]) ** -0.5)
            st[a + "out"] = mat(W, s=0.2, mean=1.0)
            delta(p + "mix.right.", L["mixer"]["right"], True)
            st[p + "mix.right.out"] = mat(W, s=0.2, mean=1.0)
        if L.get("mlp") is not None:
            F_ = L["mlp"]["ff"]
            st[p + "norm2"] = mat(s=0.1, mean=1.0)
            st[p + "mlp.gate"], st[p + "mlp.up"] = mat(F_, W, s=W ** -0.5), mat(F_, W, s=W ** -0.5)
            st[p + "mlp.down"] = mat(W, F_, s=F_ ** -0.5)
    return st


def greedy(w, cfg, prompt, steps):
    """Greedy continuation of one prompt by full recomputation; returns (tokens, their logits rows)."""
    toks, rows = list(prompt), []
    for _ in range(steps):
        z = forward(w, cfg, toks)[-1]
        rows.append(z)
        toks.append(int(torch.argmax(z)))
    return toks[len(prompt):], torch.stack(rows)
