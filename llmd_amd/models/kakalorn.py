"""Kakalorn: a decoder-only stack whose layers are listed one by one in its configuration.

Every sublayer is normed before and after (plain-weight RMS norms), and what a mixer reads first
passes a short causal convolution over time that is added to it:

    h = norm1(x);  h <- h + conv(h);  x <- x + norm1b(mixer(h));  x <- x + norm2b(ff(norm2(x)))

Mixers (models/mixers.py):
  ``attention``         grouped attention whose values are the projected keys (no value projection),
                        biased q / k, weighted query / key norms ahead of a partial half-split rotation,
                        a sliding window that keeps the sequence's first tokens, a learned sink per head
  ``hgrn2``             gated linear recurrence: forget gate f bounded below, write strength 1 - f
  ``latent_attention``  queries through a normed latent, interleaved rotary pairs with ramp-scaled
                        frequencies, one sigmoid gate per head; a layer with ``kv_from`` reads the latent
                        cache of an earlier layer with its own up-projections
Feed-forward: W_down relu(W_up h)^2, or none.

The residual and all norms are fp32 in both activation types; one kernel per sublayer norms the
sublayer's result, adds it to the residual and norms the sum for the next reader. Attention layers
cache in the paged pools (one per layer that owns a cache); the recurrences and the last inputs of
every layer's convolution live in the state pool.
"""
from __future__ import annotations

import torch

from llmd_amd.engine.attn_meta import AttnMeta
from llmd_amd.engine.config import ModelConfig
from llmd_amd.ops import seqmix as sm
from llmd_amd.parallel.state import get_state

from .layers import LMHead, VocabEmbedding
from .mixers import GroupedAttention, Hgrn2Mixer, InputConv, LatentAttention, SquaredReluMLP, _param


def make_mixer(spec: dict, d: int, eps: float, max_pos: int, device, dtype, earlier: list):
    """``earlier``: the mixers of the layers before this one (a shared latent cache names one)."""
    t, m = spec["type"], spec["mixer"]
    if t == "attention":
        mask = m.get("mask") or {}
        if m.get("vdim", m["dim"]) != m["dim"]:
            raise ValueError("attention: the values are the keys, so vdim must equal dim")
        return GroupedAttention(d, m["heads"], m["kv_heads"], m["dim"], m["dim"], m["scale"], m.get("rot"), eps,
                                max_pos, device, dtype, bias=True, interleaved=False, unit_norm=True, v_mix=False,
                                gate=False, norm_weight=True, sink="learned", v_from_k=True, norm_first=True,
                                window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0))
    if t == "hgrn2":
        return Hgrn2Mixer(d, m["heads"], m["dim"], m["vdim"], eps, device, dtype)
    if t == "latent_attention":
        rot = m["rot"]
        src = m.get("kv_from")
        return LatentAttention(d, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"],
                               rot["dims"], rot["base"], eps, max_pos, device, dtype, q_rank=m["q_rank"],
                               interleaved=True, rot_scaling=rot.get("scaling"), gate=True,
                               kv_source=None if src is None else earlier[src])
    raise ValueError(f"unknown mixer type {t!r}")


def make_mlp(m, d: int, device, dtype):
    if m is None:
        return None
    if m["kind"] == "dense":
        return SquaredReluMLP(d, m["ff"], device, dtype)
    raise ValueError(f"unknown feed-forward kind {m['kind']!r}")


class KakalornLayer(torch.nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, max_pos: int, device, dtype, earlier: list):
        super().__init__()
        spec = cfg.layer_specs[idx]
        d, eps = cfg.hidden_size, cfg.rms_norm_eps
        self.canon1 = InputConv(d, cfg.conv_taps, device, dtype)
        self.mix = make_mixer(spec, d, eps, max_pos, device, dtype, earlier)
        self.mlp = make_mlp(spec.get("mlp"), d, device, dtype)
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if self.mlp is not None else ()):
            setattr(self, n, _param((d,), device, dtype, fill=1.0))


class KakalornForCausalLM(torch.nn.Module):
    supports_float32 = True
    stateful = True  # recurrences and convolution inputs: no prefix reuse, one state slot per sequence

    def __init__(self, cfg: ModelConfig, device="cuda", max_pos: int = 32768, dtype=torch.bfloat16):
        super().__init__()
        if get_state().tp_size != 1:
            raise ValueError("kakalorn runs on one rank (its recurrent layers are not tensor-parallel)")
        self.cfg, self.dtype = cfg, dtype
        d = cfg.hidden_size
        self.embed = VocabEmbedding(cfg.vocab_size, d, device, dtype=dtype)
        self.layers = torch.nn.ModuleList()
        for i in range(cfg.num_hidden_layers):
            self.layers.append(KakalornLayer(cfg, i, max_pos, device, dtype, [l.mix for l in self.layers]))
        self.norm = _param((d,), device, dtype, fill=1.0)
        self.lm_head = LMHead(cfg.vocab_size, d, device, dtype=dtype)
        self.finalize()

    def finalize(self):
        """Derived constants (fp32 copies of biases, bounds, norm weights and sinks): after every weight load."""
        for m in self.modules():
            if m is not self and hasattr(m, "finalize"):
                m.finalize()

    def attention_layers(self):
        """The mixers that own a paged cache (a latent layer that reads another's has none)."""
        return [l.mix for l in self.layers
                if isinstance(l.mix, GroupedAttention) or (isinstance(l.mix, LatentAttention) and l.mix.owns_cache)]

    def state_layers(self):
        out = []
        for l in self.layers:
            out.append(l.canon1)
            if hasattr(l.mix, "state_shapes"):
                out.append(l.mix)
        return out

    def kv_specs(self):
        return [a.kv_spec() for a in self.attention_layers()]

    @torch.no_grad()
    def forward(self, input_ids, meta: AttnMeta, layer_out=None):
        """``layer_out``: optional list that receives a copy of the residual after every layer."""
        T, L = input_ids.shape[0], len(self.layers)
        d, eps, dt = self.cfg.hidden_size, self.cfg.rms_norm_eps, self.dtype
        x = torch.empty(T, d, dtype=torch.float32, device=input_ids.device)
        h = sm.embed_norm(input_ids, self.embed.weight, self.layers[0].norm1 if L else self.norm, eps, x, dt)
        for i, l in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < L else self.norm   # the last pass norms for the head
            y = l.mix(l.canon1(h, meta), meta)
            if l.mlp is None:
                h = sm.post_norm_add(y, l.norm1b, x, eps, dt, nxt)
            else:
                h = sm.post_norm_add(y, l.norm1b, x, eps, dt, l.norm2)
                h = sm.post_norm_add(l.mlp(h), l.norm2b, x, eps, dt, nxt)
            if layer_out is not None:
                layer_out.append(x.clone())
        return h

    @torch.no_grad()
    def compute_logits(self, h):
        # over the head's padded rows, so that the rows stay 16-byte aligned for the sampling kernel
        logits = torch.nn.functional.linear(h, self.lm_head.weight).float()
        return logits[:, :self.cfg.vocab_size]

    def weight_specs(self) -> list:
        specs = [("embed", self.embed.weight, "vocab", None), ("final.norm", self.norm, "replicate", None),
                 ("head", self.lm_head.weight, "vocab", None)]

        def add(name, p, kind="replicate", extra=None):
            specs.append((name, p, kind, extra))

        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            for n in ("norm1", "norm1b", "norm2", "norm2b"):
                if hasattr(layer, n):
                    add(pre + n, getattr(layer, n))
            add(pre + "canon1", layer.canon1.weight)
            m, mp = layer.mix, pre + "mix."
            if isinstance(m, GroupedAttention):
                off = 0
                for n, rows in (("q", m.nq), ("k", m.nk)):
                    add(mp + n, m.proj.weight, "fused", (off, 1, rows))
                    add(mp + n + ".b", m.bias, "fused", (off, 1, rows))
                    off += rows
                for n, p in (("q.norm", m.q_norm), ("k.norm", m.k_norm), ("sink", m.sink), ("o", m.o.weight)):
                    add(mp + n, p)
            elif isinstance(m, Hgrn2Mixer):
                off = 0
                for n, rows in (("q", m.nq), ("f", m.nq), ("v", m.nv)):
                    add(mp + n, m.proj.weight, "fused", (off, 1, rows))
                    off += rows
                for n, p in (("f.b", m.f_bias), ("lower", m.lower), ("norm", m.norm), ("o", m.o.weight)):
                    add(mp + n, p)
            else:
                add(mp + "dq", m.proj.weight, "fused", (0, 1, m.n_q))
                if m.owns_cache:
                    add(mp + "dkv", m.proj.weight, "fused", (m.n_q, 1, m.n_kv))
                    add(mp + "dkv.norm", m.dkv_norm)
                add(mp + "g", m.proj.weight, "fused", (m.n_q + m.n_kv, 1, m.H))
                for n, p in (("dq.norm", m.dq_norm), ("uq", m.uq.weight), ("uk", m.uk), ("uv", m.uv),
                             ("o", m.o.weight)):
                    add(mp + n, p)
            if layer.mlp is not None:
                add(pre + "mlp.up", layer.mlp.up.weight)
                add(pre + "mlp.down", layer.mlp.down.weight)
        return specs
