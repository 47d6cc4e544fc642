"""Sequence mixers and feed-forwards for per-layer stacks (models/mekusun.py): every size and
constant is an argument, so another stack can reuse them.

* ``LatentAttention``  - attention over a low-rank latent cache, any (heads, unrotated dim,
  rotated dim, value dim, latent rank); weight-absorbed, so the paged cache holds one row
  [latent | rotated shared key] per token (the fixed-size DeepSeek form is models/deepseek.py).
* ``Mamba1Mixer``      - selective state-space scan with a short causal convolution.
* ``GeneralDeltaMixer``- generalized delta rule with per-channel decay and removal rate.
* ``ActMLP`` / ``PlainMoE`` - ungated feed-forwards (xIELU dense; erf-GELU experts with a
  biased fp32 router and softmax over the chosen logits).
* ``GroupedAttention`` - grouped-query softmax attention with its own key and value sizes, biases,
  partial rotary (interleaved or half-split pairs, optional frequency scaling), unit-RMS queries and
  keys, value mixing with an earlier layer and a sigmoid output gate - each one an option.
* ``GatedMLP`` / ``ScoreMoE`` - gated feed-forwards (act(gate) * up); experts chosen by softmax
  scores plus a selection-only correction, with identity experts.
* ``GroupedAttention`` options for position-free stacks: weighted query / key norms, a distance bias
  per head, chunked visibility, a sink in the softmax's denominator, an output bias.
* ``GatedDeltaMixer``  - gated delta rule behind short convolutions, its decay one per head or one
  per head and key channel (low-rank), gate SiLU or sigmoid (low-rank).
* ``ParallelMixer``    - two mixers that read the same input, their results added with two scales.
* ``SigmoidMoE``       - gated experts chosen by sigmoid scores whose weight scales the expert's input.
* ``BigramEmbedding``  - token embedding plus a hashed (previous, current) table.
* ``GroupedAttention`` options for windowed stacks: values that are the projected keys, query / key
  norms ahead of the rotation, a sliding window that keeps the sequence's first tokens, learned sinks.
* ``LatentAttention`` options: queries through a normed latent of their own, interleaved rotary pairs,
  ramp-scaled frequencies, one sigmoid gate per head, the cache of an earlier layer instead of its own.
* ``Hgrn2Mixer``       - gated linear recurrence: forget gate f (bounded below), write strength 1 - f.
* ``SquaredReluMLP``   - W_down relu(W_up h)^2.
* ``InputConv``        - h + a short causal convolution of h, in front of a mixer.

Recurrent state lives in the engine's state pool (engine/state_cache.py): a mixer with
``state_shapes()`` gets its per-slot tensors through ``bind_state``; the step's
``AttnMeta.seq`` says which slot each run of tokens continues. Matrix products go to the
vendor GEMM through ``ops.linear``; everything between them runs in the kernels of
``ops.seqmix`` (fp32 where the recurrences, norms and scores need it).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from llmd_amd.engine.attn_meta import AttnMeta
from llmd_amd.ops import seqmix as sm

from .layers import ColumnLinear, _init_weight


def _param(shape, device, dtype, std=0.02, fill=None):
    t = torch.empty(shape, device=device, dtype=dtype)
    if fill is None:
        _init_weight(t, std)
    else:
        t.fill_(fill)
    return torch.nn.Parameter(t, requires_grad=False)


def rope_table(dims: int, base: float, max_pos: int, device, scaling=None) -> torch.Tensor:
    """[max_pos, dims] fp32 = [cos(p f_i) | sin(p f_i)], f_i = base^(-2i/dims), angles in fp64.

    ``scaling`` = {factor, low, high, original}: frequency scaling by wavelength l = 2 pi / f -
    f stays where l < original / high, becomes f / factor where l > original / low, and between
    the two is the blend (1 - s) f / factor + s f with s = (original / l - low) / (high - low).

    ``scaling`` = {factor, original, fast, slow}: the ramp form. With n(t) = dims ln(original / (2 pi t))
    / (2 ln base), the index at which a wave turns t times over ``original`` positions, lo =
    max(floor(n(fast)), 0), hi = min(ceil(n(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo,
    0.001), 0, 1) the frequency is (1 - r_i) f_i + r_i f_i / factor, and cos and sin are both
    multiplied by 0.1 ln(factor) + 1."""
    half = dims // 2
    f = torch.tensor(base, dtype=torch.float64) ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    mag = 1.0
    if scaling and "fast" in scaling:
        fac, orig = float(scaling["factor"]), float(scaling["original"])
        turn = lambda t: dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))  # noqa: E731
        lo = max(math.floor(turn(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
        r = ((torch.arange(half, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / fac * r + f * (1.0 - r)
        mag = 0.1 * math.log(fac) + 1.0
    elif scaling:
        fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wl = 2.0 * math.pi / f
        s = (orig / wl - lo) / (hi - lo)
        mid = (1.0 - s) * f / fac + s * f
        f = torch.where(wl < orig / hi, f, torch.where(wl > orig / lo, f / fac, mid))
    a = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None]
    return (torch.cat([a.cos(), a.sin()], -1) * mag).float().to(device)


class LatentAttention(torch.nn.Module):
    """Attention over a low-rank latent cache: the paged cache holds one row [normed latent | rotated
    shared key part] per token; W_uk is absorbed into the query and W_uv applied to the latent read-out.

    q_rank       > 0: queries go through a latent of their own, q = W_uq rms_norm(W_dq h) (weight
                 ``dq_norm``); the layer's input projections [dq | dkv | gate] are then ONE product
    interleaved  rotary pairs (2i, 2i+1) instead of (i, i + rot_dims/2)
    rot_scaling  frequency scaling of ``rope_table``
    gate         head h's result is multiplied by sigmoid(W_g h)_h, one number per head
    kv_source    an earlier LatentAttention whose cache this layer reads instead of writing its own
                 (no W_dkv here; W_uk, W_uv, queries and everything else are this layer's)
    """
    is_latent = True

    def __init__(self, d_model, heads, dim, rot_dim, vdim, kv_rank, scale, rot_dims, rot_base, eps, max_pos,
                 device, dtype, q_rank=0, interleaved=False, rot_scaling=None, gate=False, kv_source=None):
        super().__init__()
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError(f"rotary dims {rot_dims} do not fit the rotated part {rot_dim}")
        self.H, self.dn, self.dr, self.dv, self.R = heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.rot_dims, self.eps = float(scale), rot_dims, eps
        self.q_rank, self.interleaved, self.has_gate = int(q_rank), bool(interleaved), bool(gate)
        self._src = [kv_source] if kv_source is not None else None   # a list: not a submodule of this layer
        if kv_source is not None and (kv_source.R, kv_source.dr, kv_source._src) != (kv_rank, rot_dim, None):
            raise ValueError("a shared latent cache needs the same latent and rotated sizes and a layer that owns it")
        self.fused = self.q_rank > 0 or self.has_gate
        n_kv = 0 if kv_source is not None else kv_rank + rot_dim
        if self.fused:
            # one product of the layer input: [query latent (or queries) | latent + shared key | gate]
            self.n_q = self.q_rank if self.q_rank else heads * (dim + rot_dim)
            self.n_kv = n_kv
            n = self.n_q + n_kv + (heads if gate else 0)
            self.proj = ColumnLinear(d_model, -(-n // 8) * 8, shard=False, device=device, dtype=dtype)
            if self.q_rank:
                self.dq_norm = _param((self.q_rank,), device, dtype, fill=1.0)
                self.uq = ColumnLinear(self.q_rank, heads * (dim + rot_dim), shard=False, device=device, dtype=dtype)
        else:
            self.q = ColumnLinear(d_model, heads * (dim + rot_dim), shard=False, device=device, dtype=dtype)
            if kv_source is None:
                self.dkv = ColumnLinear(d_model, kv_rank + rot_dim, shard=False, device=device, dtype=dtype)
        if kv_source is None:
            self.dkv_norm = _param((kv_rank,), device, dtype, fill=1.0)
        self.uk = _param((heads * dim, kv_rank), device, dtype)
        self.uv = _param((heads * vdim, kv_rank), device, dtype)
        self.o = ColumnLinear(heads * vdim, d_model, shard=False, device=device, dtype=dtype)
        self.register_buffer("cos_sin", rope_table(rot_dims, rot_base, max_pos, device, rot_scaling),
                             persistent=False)
        self.cache = None
        # what the runner's generic bookkeeping reads
        self.Hq, self.Hkv, self.D, self.window, self.sinks = heads, 1, kv_rank + rot_dim, 0, None

    @property
    def owns_cache(self) -> bool:
        return self._src is None

    def kv_spec(self):
        return 1, 1, self.R + self.dr  # (planes, heads, dim): one latent row per token

    def bind_cache(self, kv_layer):
        """kv_layer [blocks, 1, 1, bs, R + dr] -> [blocks, bs, R + dr]."""
        self.cache = kv_layer[:, 0, 0]

    def forward(self, h, meta: AttnMeta):
        T, H, R, dn, dr = h.shape[0], self.H, self.R, self.dn, self.dr
        s = meta.seq
        gate = kv = None
        if self.fused:
            p = self.proj(h)
            q = self.uq(sm.rms_norm(p[:, :self.q_rank], self.dq_norm, self.eps)) if self.q_rank else p[:, :self.n_q]
            if self.n_kv:
                kv = p[:, self.n_q:self.n_q + self.n_kv]
            if self.has_gate:
                gate = p[:, self.n_q + self.n_kv:self.n_q + self.n_kv + H]
        else:
            q = self.q(h)
            if self._src is None:
                kv = self.dkv(h)
        cache = self.cache if self._src is None else self._src[0].cache
        q_abs = torch.empty(T, H, R + dr, dtype=h.dtype, device=h.device)
        sm.latent_rope_cache(q, kv, self.dkv_norm if kv is not None else None, self.eps, meta.positions, self.cos_sin,
                             H, dn, dr, self.rot_dims, R, meta.slot_mapping, cache, q_abs, self.interleaved)
        # absorb W_uk into the query: scores against the latent itself
        qn = q.reshape(T, H, dn + dr)[:, :, :dn].transpose(0, 1)                      # [H, T, dn]
        q_abs[:, :, :R].copy_(torch.bmm(qn, self.uk.view(H, dn, R)).transpose(0, 1))
        o_lat = sm.latent_attention(q_abs, cache, s.tables, s.row_seq, s.row_len, self.scale, R,
                                    rows_per_group=4 if s.max_q > 1 else 1, seq=s, gate=gate)
        o = torch.bmm(o_lat.transpose(0, 1), self.uv.view(H, self.dv, R).transpose(1, 2))  # [H, T, dv]
        return self.o(o.transpose(0, 1).reshape(T, H * self.dv))


class Mamba1Mixer(torch.nn.Module):
    def __init__(self, d_model, inner, state, dt_rank, taps, device, dtype):
        super().__init__()
        self.C, self.N, self.R, self.taps = inner, state, dt_rank, taps
        self.dtype = dtype
        self.in_proj = ColumnLinear(d_model, 2 * inner, shard=False, device=device, dtype=dtype)
        self.conv = _param((inner, taps), device, dtype, std=0.2)
        self.conv_b = _param((inner,), device, dtype, fill=0.0)
        self.x_proj = ColumnLinear(inner, dt_rank + 2 * state, shard=False, device=device, dtype=dtype)
        self.dt_proj = ColumnLinear(dt_rank, inner, shard=False, device=device, dtype=dtype)
        self.dt_b = _param((inner,), device, dtype, fill=0.0)
        self.A_log = _param((inner, state), device, dtype, fill=0.0)
        self.D = _param((inner,), device, dtype, fill=1.0)
        self.o = ColumnLinear(inner, d_model, shard=False, device=device, dtype=dtype)
        self.A = None
        self.conv_state = self.ssm_state = None

    def finalize(self):
        """After the weights are loaded: A = -exp(A_log) once, in fp32."""
        self.A = -torch.exp(self.A_log.data.float())

    def state_shapes(self):
        return [((max(self.taps - 1, 1), self.C), self.dtype), ((self.C, self.N), torch.float32)]

    def bind_state(self, tensors):
        self.conv_state, self.ssm_state = tensors

    def forward(self, h, meta: AttnMeta):
        s = meta.seq
        xz = self.in_proj(h)
        xc = sm.causal_conv_silu(xz, self.C, self.conv, self.conv_b, self.conv_state, s.seq_start, s.seq_slot,
                                 s.seq_init, s.max_q)
        bc = self.x_proj(xc)
        dt_raw = self.dt_proj(bc[:, :self.R])
        y = sm.selective_scan(xc, dt_raw, self.dt_b, self.A, bc, self.R, self.N, self.D, xz, self.C,
                              self.ssm_state, s.seq_start, s.seq_slot, s.seq_init)
        return self.o(y)


class GeneralDeltaMixer(torch.nn.Module):
    def __init__(self, d_model, heads, dim, decay_rank, eps, device, dtype):
        super().__init__()
        self.H, self.d, self.eps, self.wr = heads, dim, eps, decay_rank
        HD = heads * dim
        # one projection of the layer input: [r | k | v | g | a | decay low-rank]
        self.proj = ColumnLinear(d_model, 5 * HD + decay_rank, shard=False, device=device, dtype=dtype)
        self.a_b = _param((HD,), device, dtype, fill=0.0)
        self.w2 = ColumnLinear(decay_rank, HD, shard=False, device=device, dtype=dtype)
        self.w0 = _param((HD,), device, dtype, fill=0.0)
        self.norm = _param((HD,), device, dtype, fill=1.0)
        self.o = ColumnLinear(HD, d_model, shard=False, device=device, dtype=dtype)
        self.state = None

    def state_shapes(self):
        return [((self.H, self.d, self.d), torch.float32)]

    def bind_state(self, tensors):
        (self.state,) = tensors

    def forward(self, h, meta: AttnMeta):
        s = meta.seq
        HD = self.H * self.d
        p = self.proj(h)
        wl = self.w2(torch.tanh(p[:, 5 * HD:]))
        y = sm.gdelta_scan(p, wl, self.w0, self.a_b, self.norm, self.eps, self.H, self.d, self.state,
                           s.seq_start, s.seq_slot, s.seq_init)
        return self.o(y)


class ActMLP(torch.nn.Module):
    """W_down xielu(W_up h): the activation's two numbers are stored raw (``act``); their
    softplus forms are taken once after loading."""

    def __init__(self, d_model, ff, device, dtype):
        super().__init__()
        self.up = ColumnLinear(d_model, ff, shard=False, device=device, dtype=dtype)
        self.down = ColumnLinear(ff, d_model, shard=False, device=device, dtype=dtype)
        self.act = _param((2,), device, dtype, fill=0.0)
        self.ap = self.aq = None

    def finalize(self):
        p, q = self.act.data.double().cpu().tolist()
        sp = lambda v: max(v, 0.0) + math.log1p(math.exp(-abs(v)))  # noqa: E731
        self.ap, self.aq = sp(p), 0.5 + sp(q)

    def forward(self, h):
        return self.down(sm.xielu(self.up(h), self.ap, self.aq))


class PlainMoE(torch.nn.Module):
    """Ungated experts W_down gelu(W_up h); router logits W_r h + b in fp32, the ``top`` largest
    chosen, weights = softmax over the chosen logits."""

    def __init__(self, d_model, ff, experts, top, device, dtype):
        super().__init__()
        self.E, self.k = experts, top
        self.router = _param((experts, d_model), device, dtype)
        self.router_b = _param((experts,), device, dtype, fill=0.0)
        self.w1 = _param((experts, ff, d_model), device, dtype)
        self.w2 = _param((experts, d_model, ff), device, dtype)
        self.router32 = self.router_b32 = None

    def finalize(self):
        self.router32, self.router_b32 = self.router.data.float(), self.router_b.data.float()

    def forward(self, h):
        logits = F.linear(h.float(), self.router32, self.router_b32)
        ids, w = sm.moe_route(logits, self.k)
        return sm.moe_ffn(h, ids, w, self.w1, self.w2)


class GroupedAttention(torch.nn.Module):
    """Causal softmax attention, ``heads`` query heads over ``kv_heads`` key/value heads, key size
    ``dim`` and value size ``vdim``. One projection of the layer input gives [q | k | v | gate]; one
    kernel adds the biases, rotates, normalises, mixes the values and writes the paged cache, whose
    row per (token, kv head) is [key | value].

    rot          None, or {dims, base, scaling} for rotary positions on the first ``dims`` dimensions
    interleaved  pairs (2i, 2i+1) instead of (i, i + dims/2)
    unit_norm    divide rotated q and k by their root mean square over ``dim`` (eps inside the root)
    v_mix        value mixing: the first such layer of a step publishes its values in
                 ``shared["v_first"]``; later ones use (1 - vmix) v + vmix v_first, which is what they
                 cache
    gate         multiply the concatenated heads by sigmoid(W_g h) before the output projection
    norm_weight  the unit norms have weights ``q_norm`` / ``k_norm`` [dim], shared by the heads
    slopes       "pow2": the score of query i and key j loses 2^(-8 (h + 1) / heads) * (i - j)
    chunk        > 0: query i sees only keys j >= (i // chunk) * chunk (borders at multiples of chunk in the sequence's positions)
    sink         one more score of 0 per head in the softmax's denominator, without a value
    sink         True: one more score of 0 per head in the softmax's denominator, without a value;
                 "learned": that score is the parameter ``sink`` [heads] (it is not scaled)
    out_bias     the output projection has a bias
    v_from_k     there is no value projection: the values are the projected keys (with their bias),
                 before norm and rotation; needs vdim == dim
    norm_first   the unit norms (and their weights) come before the rotation instead of after it
    window       > 0: query i sees key j <= i only if i - j < window or j < keep_first; the kept first
                 tokens keep their own positions
    """
    is_latent = False

    def __init__(self, d_model, heads, kv_heads, dim, vdim, scale, rot, eps, max_pos, device, dtype, bias=True,
                 interleaved=True, unit_norm=True, v_mix=False, gate=True, norm_weight=False, slopes=None, chunk=0,
                 sink=False, out_bias=False, v_from_k=False, norm_first=False, window=0, keep_first=0):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads do not divide over {kv_heads} key/value heads")
        if v_from_k and (vdim != dim or v_mix):
            raise ValueError("values that are the keys need vdim == dim and no value mixing")
        if window and chunk:
            raise ValueError("a sliding window and chunks do not combine")
        self.Hq, self.Hkv, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.interleaved, self.unit_norm = float(scale), eps, interleaved, unit_norm
        self.v_mix, self.has_gate = bool(v_mix), bool(gate)
        self.v_from_k, self.norm_first = bool(v_from_k), bool(norm_first)
        self.win, self.keep_first = int(window), int(keep_first) if window else 0
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, 0 if v_from_k else kv_heads * vdim
        n = self.nq + self.nk + self.nv + (heads * vdim if gate else 0)
        self.n_out = -(-n // 8) * 8  # rows of 16-byte multiples for the vector loads downstream
        self.proj = ColumnLinear(d_model, self.n_out, shard=False, device=device, dtype=dtype)
        self.bias = _param((self.nq + self.nk + self.nv,), device, dtype, fill=0.0)
        self.has_bias = bias
        self.vmix = _param((), device, dtype, fill=0.0)
        self.o = ColumnLinear(heads * vdim, d_model, bias=bool(out_bias), shard=False, device=device, dtype=dtype)
        self.norm_weight, self.chunk = bool(norm_weight), int(chunk)
        if norm_weight:
            if not unit_norm:
                raise ValueError("norm weights need the unit norm")
            self.q_norm = _param((dim,), device, dtype, fill=1.0)
            self.k_norm = _param((dim,), device, dtype, fill=1.0)
        if slopes not in (None, "pow2"):
            raise ValueError(f"unknown distance slopes {slopes!r}")
        self.slopes = None
        if slopes == "pow2":
            self.slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=torch.float32,
                                       device=device)
        self.sink_logits = torch.zeros(heads, dtype=torch.float32, device=device) if sink else None
        if sink == "learned":
            self.sink = _param((heads,), device, dtype, fill=0.0)
        self.qk_w32 = None
        self.rot_dims = 0
        if rot:
            self.rot_dims = int(rot["dims"])
            if self.rot_dims > dim or self.rot_dims % 2:
                raise ValueError(f"rotary dims {self.rot_dims} do not fit the head size {dim}")
            self.register_buffer("cos_sin", rope_table(self.rot_dims, rot["base"], max_pos, device,
                                                       rot.get("scaling")), persistent=False)
        else:
            self.cos_sin = None
        self.cache = None
        self.bias32, self.lam = None, 0.0
        # what the runner's generic bookkeeping reads
        self.D, self.window, self.sinks = dim + vdim, 0, None

    def finalize(self):
        self.bias32 = self.bias.data.float() if self.has_bias else None
        self.lam = float(self.vmix.data.float().item())
        if self.norm_weight:
            self.qk_w32 = torch.stack([self.q_norm.data.float(), self.k_norm.data.float()]).contiguous()
        if hasattr(self, "sink"):
            self.sink_logits = self.sink.data.float()

    def kv_spec(self):
        return 1, self.Hkv, self.dim + self.vdim  # (planes, heads, row): [key | value] per kv head

    def bind_cache(self, kv_layer):
        """kv_layer [blocks, 1, Hkv, bs, dim + vdim] -> [blocks, Hkv, bs, dim + vdim]."""
        self.cache = kv_layer[:, 0]

    def forward(self, h, meta: AttnMeta, shared=None, p=None):
        """``p``: this layer's projection of h when a caller has already computed it (a row view)."""
        T = h.shape[0]
        if p is None:
            p = self.proj(h)
        q = torch.empty(T, self.Hq, self.dim, dtype=h.dtype, device=h.device)
        v_first, mode = None, 0
        if self.v_mix:
            v_first = shared.get("v_first")
            mode = 2 if v_first is not None else 1
            if v_first is not None and v_first.shape[1] != self.nv:
                raise ValueError("value mixing needs the same kv heads x value size in all layers that use it")
            if v_first is None:
                v_first = shared["v_first"] = torch.empty(T, self.nv, dtype=torch.float32, device=h.device)
        sm.qkv_rope_cache(p, self.bias32, meta.positions, self.cos_sin, self.Hq, self.Hkv, self.dim, self.vdim,
                          self.rot_dims, self.interleaved, self.eps if self.unit_norm else None, v_first, mode,
                          self.lam, meta.slot_mapping, self.cache, q, self.qk_w32, self.norm_first, self.v_from_k)
        n0 = self.nq + self.nk + self.nv
        gate = p[:, n0:n0 + self.Hq * self.vdim] if self.has_gate else None
        o = sm.grouped_attention(q, self.cache, self.dim, self.vdim, self.scale, meta.seq, gate, self.slopes,
                                 self.chunk, self.sink_logits, self.win, self.keep_first)
        return self.o(o)


class GatedMLP(torch.nn.Module):
    """W_down (act(W_gate h) * (W_up h)), gate and up as one projection; act "gelu_tanh" or "silu"."""

    def __init__(self, d_model, ff, act, device, dtype):
        super().__init__()
        self.ff, self.act = ff, act
        self.gate_up = ColumnLinear(d_model, 2 * ff, shard=False, device=device, dtype=dtype)
        self.down = ColumnLinear(ff, d_model, shard=False, device=device, dtype=dtype)

    def forward(self, h):
        return self.down(sm.gated_act(self.gate_up(h), self.ff, self.act))


class ScoreMoE(torch.nn.Module):
    """Gated experts chosen by score: router outputs over ``experts + identity`` entries in fp32,
    scores = softmax over all of them, the ``top`` largest of score + correction chosen, weights = the
    chosen scores over their sum. The last ``identity`` entries have no weights: they return their
    input."""

    def __init__(self, d_model, ff, experts, identity, top, act, device, dtype):
        super().__init__()
        self.E, self.I, self.k, self.act = experts, identity, top, act
        self.router = _param((experts + identity, d_model), device, dtype)
        self.correction = _param((experts + identity,), device, dtype, fill=0.0)
        self.w1 = _param((experts, 2 * ff, d_model), device, dtype)   # [gate rows | up rows]
        self.w2 = _param((experts, d_model, ff), device, dtype)
        self.ff = ff
        self.router32 = self.correction32 = None

    def finalize(self):
        self.router32, self.correction32 = self.router.data.float(), self.correction.data.float()

    def forward(self, h):
        logits = F.linear(h.float(), self.router32)
        ids, w = sm.moe_route_scores(logits, self.correction32, self.k)
        return sm.moe_gated_ffn(h, ids, w, self.w1, self.w2, self.act)


class GatedDeltaMixer(torch.nn.Module):
    """Gated delta rule. One projection of the layer input gives [q | k | v | beta | decay | gate]:
    ``kv_heads`` query/key heads of size ``dim`` and ``heads`` value heads of size ``vdim`` (value
    head h uses q/k head h // (heads / kv_heads)). q, k and v pass a short causal convolution per
    channel (``taps`` taps, the last one the current token's, no bias) and SiLU; the scan kernel
    makes q and k unit vectors, q times dim^-1/2, beta = sigmoid, the decay
    g = exp(-exp(A_log_h) softplus(a + dt_bias)) and runs S <- g S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q, then the head's RMS norm with ``norm`` [vdim] and the gate.

    channel=False  one decay per head (a = W_a h, [heads]); gate silu(W_g h)
    channel=True   one decay per head and key channel (a = W_a2 (W_a1 h), [heads * dim], rank
                   ``decay_rank``); gate sigmoid(W_g2 (W_g1 h)), rank ``gate_rank``

    State per sequence: the last taps - 1 inputs of the convolutions and S [heads, dim, vdim] fp32."""

    def __init__(self, d_model, heads, kv_heads, dim, vdim, taps, eps, device, dtype, channel=False, decay_rank=0,
                 gate_rank=0):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} value heads do not divide over {kv_heads} query/key heads")
        self.H, self.G, self.dk, self.dv, self.taps, self.eps = heads, kv_heads, dim, vdim, taps, eps
        self.channel, self.dtype = bool(channel), dtype
        self.nqk, self.nv = kv_heads * dim, heads * vdim
        self.C = 2 * self.nqk + self.nv
        if channel and (decay_rank <= 0 or gate_rank <= 0):
            raise ValueError("the channel form needs the ranks of its decay and gate projections")
        self.n_dec = decay_rank if channel else heads
        self.n_gate = gate_rank if channel else self.nv
        n = self.C + heads + self.n_dec + self.n_gate
        self.n_out = -(-n // 8) * 8  # rows of 16-byte multiples
        self.proj = ColumnLinear(d_model, self.n_out, shard=False, device=device, dtype=dtype)
        self.conv = _param((self.C, taps), device, dtype, std=0.2)
        self.register_buffer("conv_b", torch.zeros(self.C, device=device, dtype=dtype), persistent=False)
        self.A_log = _param((heads,), device, dtype, fill=0.0)
        self.dt_bias = _param((heads * dim if channel else heads,), device, dtype, fill=0.0)
        self.norm = _param((vdim,), device, dtype, fill=1.0)
        if channel:
            self.a2 = ColumnLinear(decay_rank, heads * dim, shard=False, device=device, dtype=dtype)
            self.g2 = ColumnLinear(gate_rank, self.nv, shard=False, device=device, dtype=dtype)
        self.o = ColumnLinear(self.nv, d_model, shard=False, device=device, dtype=dtype)
        self.A = self.dt_bias32 = None
        self.conv_state = self.state = None

    def finalize(self):
        self.A = torch.exp(self.A_log.data.float())
        self.dt_bias32 = self.dt_bias.data.float()

    def state_shapes(self):
        return [((max(self.taps - 1, 1), self.C), self.dtype), ((self.H, self.dk, self.dv), torch.float32)]

    def bind_state(self, tensors):
        self.conv_state, self.state = tensors

    def forward(self, h, meta: AttnMeta, p=None):
        """``p``: this layer's projection of h when a caller has already computed it (a row view)."""
        s = meta.seq
        if p is None:
            p = self.proj(h)
        xc = sm.causal_conv_silu(p, self.C, self.conv, self.conv_b, self.conv_state, s.seq_start, s.seq_slot,
                                 s.seq_init, s.max_q)
        c0 = self.C
        beta = p[:, c0:c0 + self.H]
        c0 += self.H
        dec = p[:, c0:c0 + self.n_dec]
        gate = p[:, c0 + self.n_dec:c0 + self.n_dec + self.n_gate]
        if self.channel:
            dec, gate = self.a2(dec), self.g2(gate)
        y = sm.gated_delta_scan(xc, self.G, self.dk, self.H, self.dv, beta, dec, self.A, self.dt_bias32, gate,
                                self.channel, self.norm, self.eps, self.state, s)
        return self.o(y)


class ParallelMixer(torch.nn.Module):
    """Two mixers side by side on the same input; the layer's result is
    left_scale * left(h) + right_scale * right(h). ``forward`` returns both results and the scales:
    the sum is taken in fp32 by the kernel that norms it and adds it to the residual."""

    def __init__(self, left, right, left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        # both read the same input: their input projections are the two row ranges of ONE weight (one
        # GEMM per layer); each mixer's own ``proj.weight`` stays a view of its rows, which is what the
        # weight loader fills
        wl, wr = left.proj.weight.data, right.proj.weight.data
        self.n_left = wl.shape[0]
        self.proj = ColumnLinear(left.proj.in_f, self.n_left + wr.shape[0], shard=False, device=wl.device,
                                 dtype=wl.dtype)
        self.proj.weight.data.copy_(torch.cat([wl, wr]))
        left.proj.weight = torch.nn.Parameter(self.proj.weight.data[:self.n_left], requires_grad=False)
        right.proj.weight = torch.nn.Parameter(self.proj.weight.data[self.n_left:], requires_grad=False)

    def forward(self, h, meta: AttnMeta):
        p = self.proj(h)
        return self.left(h, meta, p=p[:, :self.n_left]), self.right(h, meta, p=p[:, self.n_left:])


class SigmoidMoE(torch.nn.Module):
    """Gated experts W_down (act(W_gate x) * (W_up x)) chosen by score: router logits in fp32, scores
    = their sigmoids, the ``top`` largest chosen, weights = the chosen scores as they are. The weight
    multiplies the expert's INPUT: the result is sum_e expert_e(s_e h)."""

    def __init__(self, d_model, ff, experts, top, act, device, dtype):
        super().__init__()
        self.E, self.k, self.ff, self.act = experts, top, ff, act
        self.router = _param((experts, d_model), device, dtype)
        self.w1 = _param((experts, 2 * ff, d_model), device, dtype)   # [gate rows | up rows]
        self.w2 = _param((experts, d_model, ff), device, dtype)
        self.router32 = None

    def finalize(self):
        self.router32 = self.router.data.float()

    def forward(self, h):
        logits = F.linear(h.float(), self.router32)
        ids, w = sm.moe_route(logits, self.k, sigmoid=True)
        return sm.moe_gated_ffn(h, ids, w, self.w1, self.w2, self.act, scale_input=True)


class BigramEmbedding(torch.nn.Module):
    """x = table[token] * scale + bigram[(previous * mul_prev + token * mul_cur) mod buckets], the
    table's last row (number ``buckets``) for a sequence's first token; ``bigram`` None: no second
    table. The previous token of a step's first token is per-sequence state (one int32 per slot)."""

    def __init__(self, vocab, d_model, scale, bigram, device, dtype):
        super().__init__()
        from .layers import VocabEmbedding

        self.table = VocabEmbedding(vocab, d_model, device, dtype=dtype)
        self.scale = float(scale)
        self.buckets = self.mul_prev = self.mul_cur = 0
        self.bigram = None
        if bigram:
            self.buckets, self.mul_prev, self.mul_cur = (int(bigram[k]) for k in ("buckets", "mul_prev", "mul_cur"))
            self.bigram = _param((self.buckets + 1, d_model), device, dtype)
        self.prev = None

    def state_shapes(self):
        return [((1,), torch.int32)]

    def bind_state(self, tensors):
        (self.prev,) = tensors

    def forward(self, ids, meta: AttnMeta, x, out_dtype):
        """Fills the fp32 residual ``x`` [T, d]; returns it in the activation type."""
        return sm.bigram_embed(ids, self.table.weight, self.scale, self.bigram, self.buckets, self.mul_prev,
                               self.mul_cur, self.prev, meta.seq, x, out_dtype)


class Hgrn2Mixer(torch.nn.Module):
    """Gated linear recurrence per head: a row of the state that forgets with f is written with 1 - f. One
    projection of the layer input gives [q | f | v]: q = silu(.) [heads, dim], v [heads, vdim] and the
    gate f = lower + (1 - lower) sigmoid(. + f_bias) per head and channel, ``lower`` its bound from
    below. Per head, in fp32:

        S <- diag(f) S + (1 - f) v^T;  o = S^T q

    then the head's RMS norm over vdim with ``norm`` [vdim] (shared by the heads) and the output
    projection. State per sequence: S [heads, dim, vdim] fp32."""

    def __init__(self, d_model, heads, dim, vdim, eps, device, dtype):
        super().__init__()
        self.H, self.dk, self.dv, self.eps = heads, dim, vdim, eps
        self.nq, self.nv = heads * dim, heads * vdim
        self.proj = ColumnLinear(d_model, -(-(2 * self.nq + self.nv) // 8) * 8, shard=False, device=device, dtype=dtype)
        self.f_bias = _param((self.nq,), device, dtype, fill=0.0)
        self.lower = _param((self.nq,), device, dtype, fill=0.0)
        self.norm = _param((vdim,), device, dtype, fill=1.0)
        self.o = ColumnLinear(self.nv, d_model, shard=False, device=device, dtype=dtype)
        self.f_bias32 = self.lower32 = self.state = None

    def finalize(self):
        self.f_bias32, self.lower32 = self.f_bias.data.float(), self.lower.data.float()

    def state_shapes(self):
        return [((self.H, self.dk, self.dv), torch.float32)]

    def bind_state(self, tensors):
        (self.state,) = tensors

    def forward(self, h, meta: AttnMeta):
        y = sm.hgrn2_scan(self.proj(h), self.H, self.dk, self.dv, self.f_bias32, self.lower32, self.norm, self.eps,
                          self.state, meta.seq)
        return self.o(y)


class SquaredReluMLP(torch.nn.Module):
    """W_down relu(W_up h)^2."""

    def __init__(self, d_model, ff, device, dtype):
        super().__init__()
        self.up = ColumnLinear(d_model, ff, shard=False, device=device, dtype=dtype)
        self.down = ColumnLinear(ff, d_model, shard=False, device=device, dtype=dtype)

    def forward(self, h):
        return self.down(sm.relu2(self.up(h)))


class InputConv(torch.nn.Module):
    """h + conv(h): a causal convolution over time on each channel (``weight`` [channels, taps], the
    last tap meets the current token, no bias, zeros before the sequence's start). State per
    sequence: its last taps - 1 inputs."""

    def __init__(self, channels, taps, device, dtype):
        super().__init__()
        self.C, self.taps, self.dtype = channels, int(taps), dtype
        self.weight = _param((channels, self.taps), device, dtype, std=0.2)
        self.state = None

    def state_shapes(self):
        return [((max(self.taps - 1, 1), self.C), self.dtype)]

    def bind_state(self, tensors):
        (self.state,) = tensors

    def forward(self, h, meta: AttnMeta):
        return sm.input_conv(h, self.weight, self.state, meta.seq)
