"""Zumizen: a decoder-only stack whose layers are listed one by one in its configuration.

The input is the scaled token embedding plus a hashed bigram table. Every layer norms its
sublayers' OUTPUTS only; the sublayers read the residual itself:

    x <- x + norm1(mixer(x));  x <- x + norm2(ff(x))            (plain-weight RMS norms)

Mixers (models/mixers.py):
  ``parallel``       chunked grouped attention (biased projections, weighted query / key norms, no
                     rotation, a distance bias per head, a sink of score 0 in the denominator)
                     beside a gated delta rule with one decay per head and a SiLU gate; the two
                     results are added with the configuration's scales.
  ``channel_delta``  gated delta rule with one decay per head and key channel and a sigmoid gate,
                     both from low-rank projections.
Feed-forward: SiLU-gated experts chosen by sigmoid scores whose weight scales the expert's input,
or none. Logits are soft-capped: c tanh(z / c).

The residual and all norms are fp32 in both activation types; one kernel per sublayer norms the
sublayer's result, adds it to the residual and hands the next sublayer its input. Attention
layers cache in the paged pools (one per layer); the delta rules, their convolutions and the
embedding's previous token live in the state pool.
"""
from __future__ import annotations

import torch

from llmd_amd.engine.attn_meta import AttnMeta
from llmd_amd.engine.config import ModelConfig
from llmd_amd.ops import seqmix as sm
from llmd_amd.parallel.state import get_state

from .layers import LMHead
from .mixers import BigramEmbedding, GatedDeltaMixer, GroupedAttention, ParallelMixer, SigmoidMoE, _param


def _delta(m: dict, d: int, eps: float, device, dtype, channel: bool):
    if channel and ("decay_rank" not in m or "gate_rank" not in m):
        raise ValueError("channel_delta: the ranks of the decay and gate projections come from the checkpoint's "
                         "tensor shapes (ModelConfig.from_hf on the model folder) or from 'decay_rank' / 'gate_rank'")
    return GatedDeltaMixer(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], eps, device, dtype,
                           channel=channel, decay_rank=m.get("decay_rank", 0), gate_rank=m.get("gate_rank", 0))


def make_mixer(spec: dict, d: int, eps: float, max_pos: int, device, dtype):
    t, m = spec["type"], spec["mixer"]
    if t == "channel_delta":
        return _delta(m, d, eps, device, dtype, True)
    if t == "parallel":
        a = m["left"]
        left = GroupedAttention(d, a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["scale"], None, eps, max_pos,
                                device, dtype, bias=True, unit_norm=True, v_mix=False, gate=False, norm_weight=True,
                                slopes="pow2", chunk=a["mask"]["size"], sink=True, out_bias=True)
        return ParallelMixer(left, _delta(m["right"], d, eps, device, dtype, False), m["left_scale"], m["right_scale"])
    raise ValueError(f"unknown mixer type {t!r}")


def make_mlp(m, d: int, device, dtype):
    if m is None:
        return None
    if m["kind"] == "moe":
        return SigmoidMoE(d, m["expert"]["ff"], m["router"]["experts"], m["router"]["top"], "silu", device, dtype)
    raise ValueError(f"unknown feed-forward kind {m['kind']!r}")


class ZumizenLayer(torch.nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, max_pos: int, device, dtype):
        super().__init__()
        spec = cfg.layer_specs[idx]
        d, self.eps = cfg.hidden_size, cfg.rms_norm_eps
        self.mix = make_mixer(spec, d, self.eps, max_pos, device, dtype)
        self.mlp = make_mlp(spec.get("mlp"), d, device, dtype)
        self.norm1 = _param((d,), device, dtype, fill=1.0)
        if self.mlp is not None:
            self.norm2 = _param((d,), device, dtype, fill=1.0)


class ZumizenForCausalLM(torch.nn.Module):
    supports_float32 = True
    stateful = True  # delta rules and the bigram's previous token: no prefix reuse, one state slot per sequence

    def __init__(self, cfg: ModelConfig, device="cuda", max_pos: int = 32768, dtype=torch.bfloat16):
        super().__init__()
        if get_state().tp_size != 1:
            raise ValueError("zumizen runs on one rank (its recurrent layers are not tensor-parallel)")
        self.cfg, self.dtype = cfg, dtype
        d = cfg.hidden_size
        self.embed = BigramEmbedding(cfg.vocab_size, d, cfg.embedding_scale, cfg.bigram, device, dtype)
        self.layers = torch.nn.ModuleList([ZumizenLayer(cfg, i, max_pos, device, dtype)
                                           for i in range(cfg.num_hidden_layers)])
        self.norm = _param((d,), device, dtype, fill=1.0)
        self.lm_head = LMHead(cfg.vocab_size, d, device, dtype=dtype)
        self.finalize()

    def finalize(self):
        """Derived constants (fp32 copies, exp(A_log)): after every weight load."""
        for m in self.modules():
            if m is not self and hasattr(m, "finalize"):
                m.finalize()

    def attention_layers(self):
        return [l.mix.left for l in self.layers if isinstance(l.mix, ParallelMixer)]

    def state_layers(self):
        out = [self.embed]
        for l in self.layers:
            out.append(l.mix.right if isinstance(l.mix, ParallelMixer) else l.mix)
        return out

    def kv_specs(self):
        return [a.kv_spec() for a in self.attention_layers()]

    def _sublayers(self):
        """(module, norm weight, is mixer, ends its layer) of every sublayer in order."""
        out = []
        for l in self.layers:
            out.append((l.mix, l.norm1, True, l.mlp is None))
            if l.mlp is not None:
                out.append((l.mlp, l.norm2, False, True))
        return out

    @torch.no_grad()
    def forward(self, input_ids, meta: AttnMeta, layer_out=None):
        """``layer_out``: optional list that receives a copy of the residual after every layer."""
        T = input_ids.shape[0]
        d, eps, dt = self.cfg.hidden_size, self.cfg.rms_norm_eps, self.dtype
        x = torch.empty(T, d, dtype=torch.float32, device=input_ids.device)
        h = self.embed(input_ids, meta, x, dt)
        subs = self._sublayers()
        for i, (fn, w, is_mixer, ends_layer) in enumerate(subs):
            nxt = self.norm if i + 1 == len(subs) else None  # the last pass also norms for the head
            if isinstance(fn, ParallelMixer):
                yl, yr = fn(h, meta)
                h = sm.post_norm_add(yl, w, x, eps, dt, nxt, yr, fn.left_scale, fn.right_scale)
            else:
                h = sm.post_norm_add(fn(h, meta) if is_mixer else fn(h), w, x, eps, dt, nxt)
            if ends_layer and layer_out is not None:
                layer_out.append(x.clone())
        if not subs:
            h = sm.post_norm_add(torch.zeros_like(h), self.norm, x, eps, dt, self.norm)
        return h

    @torch.no_grad()
    def compute_logits(self, h):
        # over the head's padded rows, so that the rows stay 16-byte aligned for the sampling kernel
        logits = torch.nn.functional.linear(h, self.lm_head.weight).float()
        if self.cfg.logit_softcap:
            sm.softcap_(logits, self.cfg.logit_softcap)
        return logits[:, :self.cfg.vocab_size]

    def weight_specs(self) -> list:
        specs = [("embed", self.embed.table.weight, "vocab", None), ("final.norm", self.norm, "replicate", None),
                 ("head", self.lm_head.weight, "vocab", None)]

        def add(name, p, kind="replicate", extra=None):
            specs.append((name, p, kind, extra))

        if self.embed.bigram is not None:
            add("bigram", self.embed.bigram)

        def delta(m: GatedDeltaMixer, mp: str):
            w, off = m.proj.weight, 0
            for n, rows in (("q", m.nqk), ("k", m.nqk), ("v", m.nv)):
                add(mp + n, w, "fused", (off, 1, rows))
                add(mp + n + ".conv", m.conv, "fused", (off, 1, rows))
                off += rows
            parts = (("b", m.H), ("a1", m.n_dec), ("g1", m.n_gate)) if m.channel else \
                    (("b", m.H), ("a", m.n_dec), ("g", m.n_gate))
            for n, rows in parts:
                add(mp + n, w, "fused", (off, 1, rows))
                off += rows
            if m.channel:
                add(mp + "a2", m.a2.weight)
                add(mp + "g2", m.g2.weight)
            for n, p in (("A_log", m.A_log), ("dt_bias", m.dt_bias), ("norm", m.norm), ("o", m.o.weight)):
                add(mp + n, p)

        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            add(pre + "norm1", layer.norm1)
            if layer.mlp is not None:
                add(pre + "norm2", layer.norm2)
            mp = pre + "mix."
            if isinstance(layer.mix, ParallelMixer):
                a, ap = layer.mix.left, mp + "left."
                off = 0
                for n, rows in (("q", a.nq), ("k", a.nk), ("v", a.nv)):
                    add(ap + n, a.proj.weight, "fused", (off, 1, rows))
                    add(ap + n + ".b", a.bias, "fused", (off, 1, rows))
                    off += rows
                for n, p in (("q.norm", a.q_norm), ("k.norm", a.k_norm), ("o", a.o.weight), ("o.b", a.o.bias)):
                    add(ap + n, p)
                delta(layer.mix.right, mp + "right.")
            else:
                delta(layer.mix, mp)
            f, fp = layer.mlp, pre + "mlp."
            if isinstance(f, SigmoidMoE):
                add(fp + "router", f.router)
                for e in range(f.E):
                    add(f"{fp}e{e}.gate", f.w1[e, :f.ff])
                    add(f"{fp}e{e}.up", f.w1[e, f.ff:])
                    add(f"{fp}e{e}.down", f.w2[e])
        return specs
