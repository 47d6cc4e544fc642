"""A plain, slow Zumizen: every mechanism written from its equations as one function over a
whole sequence in float64, token by token where the design is recurrent. It shares no code with
llmd_amd; the tests compare the framework with it.

``cfg`` is the configuration as a dict (the layout of a config.json), ``W`` maps tensor names
to tensors.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def embed(tokens, table, scale, bigram=None, big=None):
    """table[token] * scale (+ the bigram row of (previous, current), the last row for the first token)."""
    x = table.to(F64)[tokens] * scale
    if bigram is not None:
        n = big["buckets"]
        rows = []
        for i, t in enumerate(tokens.tolist()):
            rows.append(n if i == 0 else (tokens[i - 1].item() * big["mul_prev"] + t * big["mul_cur"]) % n)
        x = x + bigram.to(F64)[torch.tensor(rows)]
    return x


def short_conv_silu(x, w):
    """Causal per-channel convolution, zeros before the start; the last column of w [C, taps]
    meets the current token."""
    T, C = x.shape
    taps = w.shape[1]
    w = w.to(F64)
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            p = t - (taps - 1 - j)
            if p >= 0:
                out[t] += w[:, j] * x[p]
    return silu(out)


def unit(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def delta_rule(q, k, v, beta, g):
    """Gated delta rule per head. q, k [T, H, dk]; v [T, H, dv]; beta [T, H]; g [T, H] (one decay per
    head) or [T, H, dk] (one per key channel: it scales the rows of S). Returns o [T, H, dv]."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        gt = g[t]
        S = S * (gt[:, :, None] if gt.dim() == 2 else gt[:, None, None])
        pred = torch.einsum("hkv,hk->hv", S, k[t])
        u = beta[t][:, None] * (v[t] - pred)
        S = S + torch.einsum("hk,hv->hkv", k[t], u)
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def delta_inputs(h, W, pre, m):
    """Projections, short convolutions, unit keys and queries, beta; shared by both delta mixers."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    lin = lambda n: h @ W[pre + n].to(F64).T  # noqa: E731
    q = short_conv_silu(lin("q"), W[pre + "q.conv"]).view(T, G, dk)
    k = short_conv_silu(lin("k"), W[pre + "k.conv"]).view(T, G, dk)
    v = short_conv_silu(lin("v"), W[pre + "v.conv"]).view(T, H, dv)
    q = unit(q) * dk ** -0.5
    k = unit(k)
    rep = H // G
    q = q.repeat_interleave(rep, 1)
    k = k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(lin("b"))
    return q, k, v, beta


def head_delta(h, W, pre, m, eps):
    """Delta rule with one decay per head, output gate silu(W_g h)."""
    T = h.shape[0]
    H, dv = m["heads"], m["vdim"]
    q, k, v, beta = delta_inputs(h, W, pre, m)
    a = h @ W[pre + "a"].to(F64).T + W[pre + "dt_bias"].to(F64)
    g = torch.exp(-torch.exp(W[pre + "A_log"].to(F64)) * softplus(a))
    o = delta_rule(q, k, v, beta, g)
    o = rms_norm(o, W[pre + "norm"], eps) * silu(h @ W[pre + "g"].to(F64).T).view(T, H, dv)
    return o.reshape(T, H * dv) @ W[pre + "o"].to(F64).T


def channel_delta(h, W, pre, m, eps):
    """Delta rule with a decay per head and key channel (low-rank projection), output gate
    sigmoid(W_g2 W_g1 h)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q, k, v, beta = delta_inputs(h, W, pre, m)
    a = (h @ W[pre + "a1"].to(F64).T) @ W[pre + "a2"].to(F64).T + W[pre + "dt_bias"].to(F64)
    g = torch.exp(-torch.exp(W[pre + "A_log"].to(F64))[None, :, None] * softplus(a).view(T, H, dk))
    o = delta_rule(q, k, v, beta, g)
    gate = torch.sigmoid((h @ W[pre + "g1"].to(F64).T) @ W[pre + "g2"].to(F64).T).view(T, H, dv)
    o = rms_norm(o, W[pre + "norm"], eps) * gate
    return o.reshape(T, H * dv) @ W[pre + "o"].to(F64).T


def chunk_attention(h, W, pre, m, eps):
    """Softmax attention inside chunks of mask.size positions, a distance bias per head, a sink of
    score 0 in the denominator, normed queries and keys, biased projections."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size = m["mask"]["size"]
    lin = lambda n: h @ W[pre + n].to(F64).T + W[pre + n + ".b"].to(F64)  # noqa: E731
    q = rms_norm(lin("q").view(T, H, dk), W[pre + "q.norm"], eps)
    k = rms_norm(lin("k").view(T, G, dk), W[pre + "k.norm"], eps)
    v = lin("v").view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        kv = hh // (H // G)
        slope = 2.0 ** (-8.0 * (hh + 1) / H)
        for i in range(T):
            lo = (i // size) * size
            js = torch.arange(lo, i + 1)
            s = (k[js, kv] @ q[i, hh]) * m["scale"] - slope * (i - js).to(F64)
            e = torch.exp(s)
            p = e / (1.0 + e.sum())
            out[i, hh] = p @ v[js, kv]
    return out.reshape(T, H * dv) @ W[pre + "o"].to(F64).T + W[pre + "o.b"].to(F64)


def moe(h, W, pre, m):
    """Sigmoid scores, the ``top`` largest chosen, the score scales the expert's INPUT."""
    E, top = m["router"]["experts"], m["router"]["top"]
    s = torch.sigmoid(h @ W[pre + "router"].to(F64).T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(s[t], top).indices.tolist():
            x = s[t, e] * h[t]
            a = silu(W[f"{pre}e{e}.gate"].to(F64) @ x) * (W[f"{pre}e{e}.up"].to(F64) @ x)
            out[t] += W[f"{pre}e{e}.down"].to(F64) @ a
    return out


def mixer(h, W, pre, spec, eps):
    m = spec["mixer"]
    if spec["type"] == "channel_delta":
        return channel_delta(h, W, pre, m, eps)
    if spec["type"] == "parallel":
        left = chunk_attention(h, W, pre + "left.", m["left"], eps)
        right = head_delta(h, W, pre + "right.", m["right"], eps)
        return m["left_scale"] * left + m["right_scale"] * right
    raise ValueError(spec["type"])


def forward(cfg, W, tokens):
    """tokens: 1-D int64. Returns (logits [T, vocab], residual after every layer [L, T, width])."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    emb = cfg.get("embedding", {})
    big = emb.get("bigram")
    x = embed(tokens, W["embed"], emb.get("scale", 1.0), W.get("bigram") if big else None, big)
    layers = []
    for i, spec in enumerate(cfg["layers"]):
        pre = f"l{i}."
        x = x + rms_norm(mixer(x, W, pre + "mix.", spec, eps), W[pre + "norm1"], eps)
        if spec.get("mlp") is not None:
            x = x + rms_norm(moe(x, W, pre + "mlp.", spec["mlp"]), W[pre + "norm2"], eps)
        layers.append(x.clone())
    z = rms_norm(x, W["final.norm"], eps) @ W["head"].to(F64).T
    cap = cfg.get("logit_softcap") or 0.0
    if cap:
        z = cap * torch.tanh(z / cap)
    return z, torch.stack(layers) if layers else x[None]


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Random tensors with the design's names and shapes (std chosen so that nothing saturates)."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(name, *shape, std=None):
        std = std if std is not None else 1.0 / math.sqrt(shape[-1])
        W[name] = (torch.randn(*shape, generator=g) * std).to(dtype)

    def vec(name, n, mean=1.0, std=0.1):
        W[name] = (mean + torch.randn(n, generator=g) * std).to(dtype)

    mat("embed", V, d, std=1.0)
    big = cfg.get("embedding", {}).get("bigram")
    if big:
        mat("bigram", big["buckets"] + 1, d, std=0.5)

    def delta(pre, m, channel):
        H, G, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        for n, rows in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
            mat(pre + n, rows, d)
            mat(pre + n + ".conv", rows, taps, std=0.6)
        mat(pre + "b", H, d)
        vec(pre + "A_log", H, mean=-0.5, std=0.5)
        vec(pre + "norm", dv)
        if channel:
            ra, rg = m.get("rank", 8), m.get("rank", 8) + 3   # two sizes that only the tensors give
            mat(pre + "a1", ra, d)
            mat(pre + "a2", H * dk, ra)
            vec(pre + "dt_bias", H * dk, mean=0.0, std=0.5)
            mat(pre + "g1", rg, d)
            mat(pre + "g2", H * dv, rg)
        else:
            mat(pre + "a", H, d)
            vec(pre + "dt_bias", H, mean=0.0, std=0.5)
            mat(pre + "g", H * dv, d)
        mat(pre + "o", d, H * dv)

    for i, spec in enumerate(cfg["layers"]):
        pre = f"l{i}."
        vec(pre + "norm1", d)
        m = spec["mixer"]
        if spec["type"] == "channel_delta":
            delta(pre + "mix.", m, True)
        else:
            a, p = m["left"], pre + "mix.left."
            for n, rows in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]),
                            ("v", a["kv_heads"] * a["vdim"])):
                mat(p + n, rows, d)
                vec(p + n + ".b", rows, mean=0.0, std=0.2)
            vec(p + "q.norm", a["dim"])
            vec(p + "k.norm", a["dim"])
            mat(p + "o", d, a["heads"] * a["vdim"])
            vec(p + "o.b", d, mean=0.0, std=0.2)
            delta(pre + "mix.right.", m["right"], False)
        f = spec.get("mlp")
        if f is not None:
            vec(pre + "norm2", d)
            mat(pre + "mlp.router", f["router"]["experts"], d, std=2.0 / math.sqrt(d))
            for e in range(f["router"]["experts"]):
                mat(f"{pre}mlp.e{e}.gate", f["expert"]["ff"], d)
                mat(f"{pre}mlp.e{e}.up", f["expert"]["ff"], d)
                mat(f"{pre}mlp.e{e}.down", d, f["expert"]["ff"])
    vec("final.norm", d)
    mat("head", V, d)
    return W
