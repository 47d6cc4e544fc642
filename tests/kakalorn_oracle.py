"""A plain, slow Kakalorn: every mechanism written from its equations as one function over a
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


def input_conv(h, w):
    """h + conv(h): causal per-channel convolution over time, zeros before the start; the last
    column of w [C, taps] meets the current token."""
    T, C = h.shape
    taps = w.shape[1]
    w = w.to(F64)
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            p = t - (taps - 1 - j)
            if p >= 0:
                out[t] += w[:, j] * h[p]
    return out


def frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` (factor, original, fast, slow) the
    long-wavelength end is divided by ``factor`` along a linear ramp. Returns (f, magnitude): cos
    and sin are multiplied by the magnitude."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    if not scaling:
        return f, 1.0
    fac, orig = float(scaling["factor"]), float(scaling["original"])

    def turn(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F64)
    return f / fac * ramp + f * (1.0 - ramp), 0.1 * math.log(fac) + 1.0


def rotate(x, pos, dims, base, interleaved, scaling=None):
    """Rotary positions on the first ``dims`` entries of the last axis of x [T, ..., n]; pairs
    (i, i + dims/2) or, interleaved, (2i, 2i + 1)."""
    f, mag = frequencies(dims, base, scaling)
    a = pos.to(F64)[:, None] * f[None]                        # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (a.cos() * mag).view(shape), (a.sin() * mag).view(shape)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def visible(i, j, size=None, keep_first=0):
    """Does position i see position j: causal, and inside the window or among the kept first ones."""
    if j > i:
        return False
    return size is None or i - j < size or j < keep_first


def softmax_attention(q, k, v, scale, group, size=None, keep_first=0, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads kv head h // group. ``sink`` [H]:
    one more term exp(sink_h) in the denominator."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // group
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, size, keep_first)]
            s = (k[js, g] @ q[i, h]) * scale
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h].to(F64))
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h].to(F64) - m) if sink is not None else 0.0)
            out[i, h] = ((e / den)[:, None] * v[js, g]).sum(0)
    return out


def attention(h, W, pre, m, eps):
    """Windowed grouped attention whose values are the projected keys."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W[pre + "q"].to(F64).T + W[pre + "q.b"].to(F64)).view(T, H, d)
    k = (h @ W[pre + "k"].to(F64).T + W[pre + "k.b"].to(F64)).view(T, G, d)
    v = k.clone()
    q, k = rms_norm(q, W[pre + "q.norm"], eps), rms_norm(k, W[pre + "k.norm"], eps)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate(q, pos, rot["dims"], rot["base"], False, rot.get("scaling"))
        k = rotate(k, pos, rot["dims"], rot["base"], False, rot.get("scaling"))
    mask = m.get("mask") or {}
    o = softmax_attention(q, k, v, m["scale"], H // G, mask.get("size"), mask.get("keep_first", 0),
                          W.get(pre + "sink"))
    return o.reshape(T, H * d) @ W[pre + "o"].to(F64).T


def hgrn2_recurrence(q, f, v):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t per head. q, f [T, H, d]; v [T, H, dv]."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F64)
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def hgrn2(h, W, pre, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    z = h @ W[pre + "q"].to(F64).T
    q = (z * torch.sigmoid(z)).view(T, H, d)
    v = (h @ W[pre + "v"].to(F64).T).view(T, H, dv)
    low = W[pre + "lower"].to(F64)
    f = (low + (1.0 - low) * torch.sigmoid(h @ W[pre + "f"].to(F64).T + W[pre + "f.b"].to(F64))).view(T, H, d)
    o = rms_norm(hgrn2_recurrence(q, f, v), W[pre + "norm"], eps)
    return o.reshape(T, H * dv) @ W[pre + "o"].to(F64).T


def latent_kv(h, W, pre, m, eps):
    """The cached part of a latent-attention layer: the normed latent and the rotated shared key."""
    R, rot = m["kv_rank"], m["rot"]
    kv = h @ W[pre + "dkv"].to(F64).T
    c = rms_norm(kv[:, :R], W[pre + "dkv.norm"], eps)
    kr = rotate(kv[:, R:], torch.arange(h.shape[0]), rot["dims"], rot["base"], True, rot.get("scaling"))
    return c, kr


def latent_attention(h, W, pre, m, eps, kv):
    """``kv`` = (latent, rotated key part) of this layer or of the layer it reads them from."""
    T = h.shape[0]
    H, d, dr, dv, rot = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["rot"]
    c, kr = kv
    cq = rms_norm(h @ W[pre + "dq"].to(F64).T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].to(F64).T).view(T, H, d + dr)
    qr = rotate(q[..., d:], torch.arange(T), rot["dims"], rot["base"], True, rot.get("scaling"))
    k = torch.cat([(c @ W[pre + "uk"].to(F64).T).view(T, H, d), kr[:, None, :].expand(T, H, dr)], -1)
    v = (c @ W[pre + "uv"].to(F64).T).view(T, H, dv)
    o = softmax_attention(torch.cat([q[..., :d], qr], -1), k, v, m["scale"], 1)
    gate = torch.sigmoid(h @ W[pre + "g"].to(F64).T)          # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * dv) @ W[pre + "o"].to(F64).T


def feed_forward(h, W, pre, m):
    if m["kind"] != "dense":
        raise ValueError(m["kind"])
    a = torch.relu(h @ W[pre + "up"].to(F64).T)
    return (a * a) @ W[pre + "down"].to(F64).T


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` receives the residual after every layer."""
    eps = cfg["norm"]["eps"]
    x = W["embed"].to(F64)[torch.as_tensor(tokens)]
    kvs = {}
    for i, l in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", l["mixer"]
        h = input_conv(rms_norm(x, W[pre + "norm1"], eps), W[pre + "canon1"])
        if l["type"] == "attention":
            y = attention(h, W, pre + "mix.", m, eps)
        elif l["type"] == "hgrn2":
            y = hgrn2(h, W, pre + "mix.", m, eps)
        elif l["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = latent_kv(h, W, pre + "mix.", m, eps)
            y = latent_attention(h, W, pre + "mix.", m, eps, kvs[i if src is None else src])
        else:
            raise ValueError(l["type"])
        x = x + rms_norm(y, W[pre + "norm1b"], eps)
        if l.get("mlp"):
            y = feed_forward(rms_norm(x, W[pre + "norm2"], eps), W, pre + "mlp.", l["mlp"])
            x = x + rms_norm(y, W[pre + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].to(F64).T


def random_weights(cfg, seed=0, dtype=torch.float32):
    """Random tensors with the design's names and shapes (std chosen so that nothing saturates)."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]
    taps = cfg["canon"]["taps"]
    W = {}

    def mat(name, *shape, std=None):
        std = std if std is not None else 1.0 / math.sqrt(shape[-1])
        W[name] = (torch.randn(*shape, generator=g) * std).to(dtype)

    def vec(name, n, mean=1.0, std=0.1):
        W[name] = (mean + torch.randn(n, generator=g) * std).to(dtype)

    mat("embed", V, d, std=1.0)
    for i, spec in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", spec["mixer"]
        vec(pre + "norm1", d)
        vec(pre + "norm1b", d)
        mat(pre + "canon1", d, taps, std=0.4)
        mp = pre + "mix."
        if spec["type"] == "attention":
            H, G, dim = m["heads"], m["kv_heads"], m["dim"]
            mat(mp + "q", H * dim, d)
            mat(mp + "k", G * dim, d)
            vec(mp + "q.b", H * dim, mean=0.0, std=0.3)
            vec(mp + "k.b", G * dim, mean=0.0, std=0.3)
            vec(mp + "q.norm", dim, std=0.3)
            vec(mp + "k.norm", dim, std=0.3)
            vec(mp + "sink", H, mean=0.0, std=1.0)
            mat(mp + "o", d, H * dim)
        elif spec["type"] == "hgrn2":
            H, dim, dv = m["heads"], m["dim"], m["vdim"]
            mat(mp + "q", H * dim, d)
            mat(mp + "f", H * dim, d)
            vec(mp + "f.b", H * dim, mean=0.5, std=1.0)
            W[mp + "lower"] = torch.rand(H * dim, generator=g).to(dtype)
            mat(mp + "v", H * dv, d)
            vec(mp + "norm", dv)
            mat(mp + "o", d, H * dv)
        else:
            H, dim, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            mat(mp + "dq", Q, d)
            vec(mp + "dq.norm", Q)
            mat(mp + "uq", H * (dim + dr), Q)
            if m.get("kv_from") is None:
                mat(mp + "dkv", R + dr, d)
                vec(mp + "dkv.norm", R)
            mat(mp + "uk", H * dim, R)
            mat(mp + "uv", H * dv, R)
            mat(mp + "g", H, d)
            mat(mp + "o", d, H * dv)
        if spec.get("mlp"):
            vec(pre + "norm2", d)
            vec(pre + "norm2b", d)
            mat(pre + "mlp.up", spec["mlp"]["ff"], d)
            mat(pre + "mlp.down", d, spec["mlp"]["ff"])
    vec("final.norm", d)
    mat("head", V, d)
    return W
