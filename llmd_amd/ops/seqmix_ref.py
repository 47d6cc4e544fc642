"""CPU implementations (plain torch, fp32 math) of the ops in ``llmd_amd.ops.seqmix``.

They exist so that the engine, its scheduler and its state manager run in CPU CI; GPU tensors
never come here. Arguments are the ones of the wrappers in ``seqmix.py``.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def _zc(x, w, eps):
    x = x.float()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float())


def embed_scale(ids, table, scale, hist):
    x = table[ids].float() * scale
    hist[0].copy_(x)
    hist[1].copy_(x)


def zc_norm(x, w, eps, out_dtype):
    return _zc(x, w, eps).to(out_dtype)


def add_post_norm(y, w_post, ls, x, eps, next_w, out_dtype):
    x.add_(_zc(y, w_post, eps) * ls.float())
    return None if next_w is None else _zc(x, next_w, eps).to(out_dtype)


def depth_avg_norm(hist, n, coef, dst, norm_w, eps, out_dtype):
    x = (hist[:n] * coef[:n].float().view(n, 1, 1)).sum(0)
    hist[dst].copy_(x)
    return _zc(x, norm_w, eps).to(out_dtype)


def _rot(v, cs, dims):
    half = dims // 2
    c, s = cs[..., :half], cs[..., half:]
    a, b = v[..., :half].float(), v[..., half:dims].float()
    return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:].float()], -1)


def _rot_pairs(v, cs, dims):
    """Pairs (2i, 2i+1) of the first ``dims`` entries."""
    half = dims // 2
    c, s = cs[..., :half], cs[..., half:]
    a, b = v[..., 0:dims:2].float(), v[..., 1:dims:2].float()
    r = torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)
    return torch.cat([r, v[..., dims:].float()], -1)


def latent_rope_cache(q, kv, norm_w, eps, positions, cos_sin, H, dn, dr, rot_dims, R, slots, cache, q_abs,
                      interleaved=False):
    T = q.shape[0]
    rot = _rot_pairs if interleaved else _rot
    cs = cos_sin[positions]                                  # [T, rot_dims]
    qr = rot(q.reshape(T, H, dn + dr)[..., dn:], cs[:, None], rot_dims)
    q_abs.view(T, H, R + dr)[..., R:] = qr.to(q_abs.dtype)
    if kv is None:
        return
    c = kv[:, :R].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    row = torch.cat([c, rot(kv[:, R:], cs, rot_dims)], -1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, R + dr)[slots[ok]] = row[ok]


def latent_attention(q_abs, cache, tables, row_seq, row_len, scale, R, out, gate=None):
    T, H, Dk = q_abs.shape
    bs = cache.shape[1]
    flat = cache.view(-1, Dk)
    for t in range(T):
        n = int(row_len[t])
        bt = tables[int(row_seq[t])].long()
        idx = bt[torch.arange(n) // bs] * bs + torch.arange(n) % bs
        K = flat[idx].float()                               # [n, Dk]
        s = (q_abs[t].float() @ K.T) * scale
        p = torch.softmax(s, -1)
        o = p @ K[:, :R]
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float())[:, None]
        out[t] = o.to(out.dtype)
    return out


def causal_conv_silu(xz, C, w, b, conv_state, seq_start, seq_slot, seq_init, out):
    taps = w.shape[1]
    wf, bf = w.float(), b.float()
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        x = xz[lo:hi, :C].float()
        prev = conv_state[sl, :taps - 1].float() if int(seq_init[i]) else torch.zeros(taps - 1, C)
        xp = torch.cat([prev, x])
        acc = bf.expand(hi - lo, C).clone()
        for j in range(taps):
            acc += xp[j:j + hi - lo] * wf[:, j]
        out[lo:hi] = F.silu(acc).to(out.dtype)
        if taps > 1:
            conv_state[sl] = xp[-(taps - 1):].to(conv_state.dtype)
    return out


def selective_scan(xc, dt_raw, dt_bias, A, bc, R, N, D, xz, C, state, seq_start, seq_slot, seq_init, out):
    Df, bias = D.float(), dt_bias.float()
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        S = state[sl].clone() if int(seq_init[i]) else torch.zeros_like(state[sl])
        for t in range(lo, hi):
            dt = F.softplus(dt_raw[t].float() + bias)
            x = xc[t].float()
            Bt, Ct = bc[t, R:R + N].float(), bc[t, R + N:R + 2 * N].float()
            S = torch.exp(dt[:, None] * A) * S + (dt * x)[:, None] * Bt[None]
            y = S @ Ct + Df * x
            out[t] = (y * F.silu(xz[t, C:].float())).to(out.dtype)
        state[sl] = S
    return out


DECAY_K = math.exp(-0.5)


def gdelta_scan(proj, wl, w0, a_b, norm_w, eps, H, d, state, seq_start, seq_slot, seq_init, out):
    HD = H * d
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        S = state[sl].clone() if int(seq_init[i]) else torch.zeros_like(state[sl])
        for t in range(lo, hi):
            p = proj[t].float()
            r, k, v, g, al = (p[j * HD:(j + 1) * HD].view(H, d) for j in range(5))
            w = torch.exp(-DECAY_K * torch.sigmoid(wl[t].float() + w0.float())).view(H, d)
            a = torch.sigmoid(al + a_b.float().view(H, d))
            u = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
            uS = torch.einsum("hi,hij->hj", u, S)
            S = w[:, :, None] * S - (a * u)[:, :, None] * uS[:, None] + k[:, :, None] * v[:, None]
            o = torch.einsum("hij,hi->hj", S, r)
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
            out[t] = (o * norm_w.float().view(H, d) * torch.sigmoid(g)).reshape(HD).to(out.dtype)
        state[sl] = S
    return out


def xielu(z, ap, aq):
    zf = z.float()
    return torch.where(zf > 0, ap * zf * zf + 0.5 * zf, aq * (torch.expm1(zf) - zf) + 0.5 * zf).to(z.dtype)


def moe_route(logits, k, sigmoid=False):
    top, ids = logits.float().topk(k, -1)
    return ids.int(), torch.sigmoid(top) if sigmoid else torch.softmax(top, -1)


def moe_ffn(h, ids, w, w1, w2):
    out = torch.zeros(h.shape, dtype=torch.float32)
    hf = h.float()
    for e in ids.unique().tolist():
        t, j = (ids == e).nonzero(as_tuple=True)
        a = F.gelu((hf[t] @ w1[e].float().T).to(h.dtype).float()).to(h.dtype).float()
        out.index_add_(0, t, (a @ w2[e].float().T) * w[t, j, None])
    return out.to(h.dtype)


def softcap_(logits, cap):
    return logits.copy_(cap * torch.tanh(logits / cap))


# ---- hyper-connected streams, grouped attention with separate key / value sizes, gated feed-forwards
def _ln(u, w, eps):
    u = u.float()
    dev = u - u.mean(-1, keepdim=True)
    return dev * torch.rsqrt(dev.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def hyper_embed(ids, table, X):
    X.copy_(table[ids].float().unsqueeze(0).expand_as(X))


def hyper_norm(X, w_in, norm_w, eps, out_dtype):
    return _ln((X * w_in.view(-1, 1, 1)).sum(0), norm_w, eps).to(out_dtype)


def hyper_update_norm(X, y, mix, w_out, next_in, next_w, eps, out_dtype):
    new = torch.einsum("st,snd->tnd", mix, X) + w_out.view(-1, 1, 1) * y.float().unsqueeze(0)
    X.copy_(new)
    return None if next_w is None else hyper_norm(X, next_in, next_w, eps, out_dtype)


def qkv_rope_cache(qkv, bias, positions, cos_sin, Hq, Hkv, dim, vdim, rot_dims, interleaved, unit_eps, v_first,
                   v_mode, lam, slots, cache, q_out, qk_w=None, norm_first=False, v_from_k=False):
    T = qkv.shape[0]
    nq, nk, nv = Hq * dim, Hkv * dim, 0 if v_from_k else Hkv * vdim
    x = qkv[:, :nq + nk + nv].float()
    if bias is not None:
        x = x + bias.float()
    q, k = x[:, :nq].view(T, Hq, dim), x[:, nq:nq + nk].view(T, Hkv, dim)
    v = k if v_from_k else x[:, nq + nk:].view(T, Hkv, vdim)

    def unit(q, k):
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + unit_eps)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + unit_eps)
        if qk_w is not None:
            q, k = q * qk_w[0].float(), k * qk_w[1].float()
        return q, k

    if unit_eps is not None and norm_first:
        q, k = unit(q, k)
    if rot_dims:
        half = rot_dims // 2
        cs = cos_sin[positions]
        c, s = cs[:, None, :half], cs[:, None, half:]

        def rot(t):
            if interleaved:
                a, b = t[..., 0:rot_dims:2], t[..., 1:rot_dims:2]
                r = torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)
            else:
                a, b = t[..., :half], t[..., half:rot_dims]
                r = torch.cat([a * c - b * s, b * c + a * s], -1)
            return torch.cat([r, t[..., rot_dims:]], -1)

        q, k = rot(q), rot(k)
    if unit_eps is not None and not norm_first:
        q, k = unit(q, k)
    if v_mode == 1:
        v_first.copy_(v.reshape(T, nv))
    elif v_mode == 2:
        v = (1.0 - lam) * v + lam * v_first.view(T, Hkv, vdim)
    q_out.copy_(q.to(q_out.dtype))
    nb, _, bs, _ = cache.shape
    kc, vc = kv_views(cache, dim, vdim)
    ok = slots >= 0
    sl = slots[ok]
    kc[sl // bs, :, sl % bs] = k[ok].to(cache.dtype)
    vc[sl // bs, :, :, sl % bs] = v[ok].to(cache.dtype)


def kv_views(cache, dim, vdim):
    """The two parts of a page [Hkv, bs * (dim + vdim)] of the grouped-attention cache: keys
    [blocks, Hkv, bs, dim] row-major, then values transposed [blocks, Hkv, vdim, bs] (a value
    column's keys are contiguous, which is how the matrix cores read them)."""
    nb, Hkv, bs, Dr = cache.shape
    flat = cache.view(nb, Hkv, bs * Dr)
    return flat[:, :, :bs * dim].view(nb, Hkv, bs, dim), flat[:, :, bs * dim:].view(nb, Hkv, vdim, bs)


def grouped_attention(q, cache, dim, vdim, tables, row_seq, row_len, scale, gate, out, slopes=None, chunk=0,
                      sinks=None, window=0, keep_first=0):
    T, Hq, _ = q.shape
    nb, Hkv, bs, _ = cache.shape
    G = Hq // Hkv
    kc, vc = kv_views(cache, dim, vdim)
    for t in range(T):
        n = int(row_len[t])
        lo = ((n - 1) // chunk) * chunk if chunk else 0       # the first key of the query's chunk
        bt = tables[int(row_seq[t])].long()
        ar = torch.arange(lo, n)
        if window:                                             # the kept first tokens and the window
            ar = ar[(ar >= n - window) | (ar < keep_first)]
        K = kc[bt[ar // bs], :, ar % bs].float()              # [n - lo, Hkv, dim]
        V = vc[bt[ar // bs], :, :, ar % bs].float()           # [n - lo, Hkv, vdim]
        qt = q[t].float().view(Hkv, G, dim)
        s = torch.einsum("hgd,nhd->hgn", qt, K) * scale
        if slopes is not None:
            s = s - slopes.float().view(Hkv, G, 1) * (n - 1 - ar).float()
        if sinks is not None:                                   # one more score per head, without a value
            s = torch.cat([s, sinks.float().view(Hkv, G, 1)], -1)
        p = torch.softmax(s, -1)[..., :ar.numel()]
        o = torch.einsum("hgn,nhv->hgv", p, V).reshape(Hq * vdim)
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float())
        out[t] = o.to(out.dtype)
    return out


def _act(z, kind):
    return F.gelu(z, approximate="tanh") if kind == "gelu_tanh" else F.silu(z)


def gated_act(gu, Fh, kind):
    return (_act(gu[:, :Fh].float(), kind) * gu[:, Fh:2 * Fh].float()).to(gu.dtype)


def moe_route_scores(logits, correction, k):
    s = torch.softmax(logits.float(), -1)
    ids = (s + correction.float()).topk(k, -1).indices
    w = torch.gather(s, 1, ids)
    return ids.int(), w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_gated_ffn(h, ids, w, w1, w2, kind, scale_input=False):
    """w1 [E, 2F, d] = [gate | up] rows, w2 [E, d, F]; ids >= E are identity experts."""
    if scale_input:
        E, F2, _ = w1.shape
        out = torch.zeros(h.shape, dtype=torch.float32)
        hf = h.float()
        for e in ids.unique().tolist():
            t, j = (ids == e).nonzero(as_tuple=True)
            gu = (hf[t] @ w1[e].float().T) * w[t, j, None]
            a = (_act(gu[:, :F2 // 2], kind) * gu[:, F2 // 2:]).to(h.dtype).float()
            out.index_add_(0, t, (a @ w2[e].float().T).to(h.dtype).float())
        return out.to(h.dtype)
    E, F2, _ = w1.shape
    out = torch.zeros(h.shape, dtype=torch.float32)
    hf = h.float()
    for e in ids.unique().tolist():
        t, j = (ids == e).nonzero(as_tuple=True)
        if e >= E:
            out.index_add_(0, t, hf[t] * w[t, j, None])
            continue
        gu = (hf[t] @ w1[e].float().T)
        a = (_act(gu[:, :F2 // 2], kind) * gu[:, F2 // 2:]).to(h.dtype).float()
        out.index_add_(0, t, (a @ w2[e].float().T).to(h.dtype).float() * w[t, j, None])
    return out.to(h.dtype)


# ---- bigram embedding, post-norm residual, gated delta rule
def bigram_embed(ids, table, scale, bigram, buckets, mul_prev, mul_cur, prev_state, seq_start, seq_slot, seq_init,
                 x, out_dtype):
    x.copy_(table[ids].float() * scale)
    rows = torch.empty_like(ids)
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        if hi == lo:
            continue
        if bigram is not None:
            prev = torch.cat([prev_state[sl].view(1).long(), ids[lo:hi - 1]])
            rows[lo:hi] = (prev * mul_prev + ids[lo:hi] * mul_cur) % buckets
            if not int(seq_init[i]):
                rows[lo] = buckets
        prev_state[sl] = ids[hi - 1]
    if bigram is not None:
        x.add_(bigram[rows].float())
    return x.to(out_dtype)


def _rms(y, eps):
    return y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)


def post_norm_add(y, w_post, x, eps, out_dtype, next_w=None, y2=None, a=1.0, b=1.0, bias=None):
    v = a * y.float()
    if y2 is not None:
        v = v + b * y2.float()
    if bias is not None:
        v = v + bias.float()
    x.add_(_rms(v, eps) * w_post.float())
    return (x if next_w is None else _rms(x, eps) * next_w.float()).to(out_dtype)


def gated_delta_scan(xc, G, dk, H, dv, beta_raw, decay_raw, A, dt_bias, gate_raw, gate_sigmoid, norm_w, eps, state,
                     seq_start, seq_slot, seq_init, out):
    T = xc.shape[0]
    nq = G * dk
    rep = H // G
    per_channel = decay_raw.shape[1] == H * dk
    qa, ka = xc[:, :nq].float().view(T, G, dk), xc[:, nq:2 * nq].float().view(T, G, dk)
    va = xc[:, 2 * nq:2 * nq + H * dv].float().view(T, H, dv)
    qa = qa * torch.rsqrt(qa.pow(2).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    ka = ka * torch.rsqrt(ka.pow(2).sum(-1, keepdim=True) + 1e-6)
    qa, ka = qa.repeat_interleave(rep, 1), ka.repeat_interleave(rep, 1)
    beta = torch.sigmoid(beta_raw.float())
    sp = F.softplus(decay_raw.float() + dt_bias.float())
    dec = torch.exp(-(A.float().view(H, 1) * sp.view(T, H, -1)))       # [T, H, dk or 1]
    gt = gate_raw.float().view(T, H, dv)
    gt = torch.sigmoid(gt) if gate_sigmoid else F.silu(gt)
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        S = state[sl].clone() if int(seq_init[i]) else torch.zeros_like(state[sl])
        for t in range(lo, hi):
            S = S * dec[t][:, :, None]
            u = beta[t][:, None] * (va[t] - torch.einsum("hkv,hk->hv", S, ka[t]))
            S = S + ka[t][:, :, None] * u[:, None]
            o = torch.einsum("hkv,hk->hv", S, qa[t])
            o = _rms(o, eps) * norm_w.float() * gt[t]
            out[t] = o.reshape(H * dv).to(out.dtype)
        if hi > lo:
            state[sl] = S
    del per_channel
    return out


# ---- embedding with the first norm, plain norms, input convolution, squared ReLU, HGRN2
def embed_norm(ids, table, w, eps, x, out_dtype):
    x.copy_(table[ids].float())
    return (_rms(x, eps) * w.float()).to(out_dtype)


def rms_norm(y, w, eps):
    return (_rms(y.float(), eps) * w.float()).to(y.dtype)


def input_conv(h, w, state, seq_start, seq_slot, seq_init, out):
    C, taps = w.shape
    wf = w.float()
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        if hi == lo:
            continue
        x = h[lo:hi].float()
        prev = state[sl, :taps - 1].float() if int(seq_init[i]) else torch.zeros(taps - 1, C)
        xp = torch.cat([prev, x])
        acc = x.clone()
        for j in range(taps):
            acc += xp[j:j + hi - lo] * wf[:, j]
        out[lo:hi] = acc.to(out.dtype)
        if taps > 1:
            state[sl, :taps - 1] = xp[-(taps - 1):].to(state.dtype)
    return out


def relu2(z):
    a = torch.relu(z.float())
    return (a * a).to(z.dtype)


def hgrn2_scan(p, H, dk, dv, f_bias, lower, norm_w, eps, state, seq_start, seq_slot, seq_init, out):
    T = p.shape[0]
    nq = H * dk
    q = F.silu(p[:, :nq].float()).view(T, H, dk)
    low = lower.float()
    f = (low + (1.0 - low) * torch.sigmoid(p[:, nq:2 * nq].float() + f_bias.float())).view(T, H, dk)
    v = p[:, 2 * nq:2 * nq + H * dv].float().view(T, H, dv)
    for i in range(seq_slot.numel()):
        lo, hi, sl = int(seq_start[i]), int(seq_start[i + 1]), int(seq_slot[i])
        if hi == lo:
            continue
        S = state[sl].clone() if int(seq_init[i]) else torch.zeros_like(state[sl])
        for t in range(lo, hi):
            S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None]
            o = torch.einsum("hkv,hk->hv", S, q[t])
            out[t] = (_rms(o, eps) * norm_w.float()).reshape(H * dv).to(out.dtype)
        state[sl] = S
    return out
