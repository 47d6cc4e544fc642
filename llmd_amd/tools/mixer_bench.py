"""Prefill and decode throughput of per-layer stacks at sizes that resemble a real model's
layers (random weights), beside the closest existing model at equal size.

``python bench.py --mixer-bench`` runs it; the default bench workload is unchanged. Three
Mekusun stacks of DeepSeek-V2-Lite's width (2048) are timed through the runner's own step
(``ModelRunner.run_plan``: the kernels, cache writes and state updates of serving):

  latent+moe : latent attention 16 heads x (128 + 64), value 128, latent 512; 64 experts, 6 chosen,
               ff 1408 - the geometry of DeepSeek-V2-Lite's layers, which run beside it
               (models/deepseek.py: MLA kernels of fixed size, gated experts + shared expert)
  mamba      : selective scan, inner 4096, state 16, dt rank 128, 4 taps; dense ff 5632
  delta      : generalized delta rule, 32 heads x 64; dense ff 5632

Two Negunex stacks (grouped attention with value mixing and an output gate over two
hyper-connected streams) run beside the existing models of the same layer geometry:

  negunex-dense : width 4096, 32 heads / 8 kv heads x 128, value 128, dense ff 14336 - beside
                  Llama-3-8B layers (models/llama.py)
  negunex-moe   : width 2048, 32 heads / 4 kv heads x 128, 128 experts + 4 identity, 8 chosen, ff 768 -
                  beside Qwen3-30B-A3B layers (models/moe_llama.py)

Two Zumizen stacks (post-norm residual, bigram embedding, experts whose score scales their input):

  zumizen-channel  : width 2048, gated delta rule 32 heads x 64 (key) x 64 (value) with a decay per key
                     channel, 4 taps; 64 experts, 6 chosen, ff 1408 - beside Mekusun's ``delta``
                     (same heads and sizes) and ``latent+moe`` (same experts)
  zumizen-parallel : width 2048, chunked attention 32 heads / 4 kv heads x 128 (chunks of 1024, distance
                     bias, sink) beside a gated delta rule 16 heads / 8 q-k heads x 128 x 128; 128 experts,
                     8 chosen, ff 768 - beside ``negunex-moe`` (same attention and expert geometry)

Four Kakalorn stacks (norms before and after every sublayer, a short convolution in front of every
mixer, squared-ReLU feed-forwards):

  kakalorn-window : width 4096, windowed attention 32 heads / 8 kv heads x 128 whose values are its keys
                    (window 1024, 4 kept first tokens, learned sinks), dense ff 14336 - beside
                    ``negunex-dense`` and Llama-3-8B layers (same heads and feed-forward size)
  kakalorn-latent : width 2048, latent attention 16 heads x (128 + 64), value 128, latent 512, query
                    latent 1536, head gates; dense ff 5632 - beside Mekusun's ``latent+moe`` (same attention)
  kakalorn-hgrn2  : width 2048, HGRN2 32 heads x 64 (key) x 64 (value); dense ff 5632 - beside Mekusun's
                    ``delta`` and ``zumizen-channel`` (same heads and sizes)
  kakalorn-hybrid : width 2048, the three mixers in turn plus a latent layer that reads the other's cache

Prefill: one prompt of ``--tokens`` tokens in one step. Decode: ``--batch`` sequences with that
context, one token each. One JSON line with tokens/s and ms per layer for every entry.
"""
from __future__ import annotations

import argparse
import json
import math
import time

import numpy as np
import torch

WIDTH = 2048


def _attn():
    return {"type": "latent_attention",
            "mixer": {"heads": 16, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "scale": 192 ** -0.5,
                      "rot": {"dims": 64, "base": 10000.0}},
            "mlp": {"kind": "moe", "expert": {"ff": 1408}, "router": {"experts": 64, "top": 6}}}


def _mamba():
    return {"type": "mamba1", "mixer": {"inner": 4096, "state": 16, "dt_rank": 128, "conv": 4},
            "mlp": {"kind": "dense", "ff": 5632}}


def _delta():
    return {"type": "general_delta", "mixer": {"heads": 32, "dim": 64, "decay_rank": 64},
            "mlp": {"kind": "dense", "ff": 5632}}


def stack_config(layer: dict, n_layers: int):
    from llmd_amd.engine.config import mekusun_config

    return mekusun_config({"architecture": "Mekusun", "width": WIDTH, "vocab": 32000, "embedding": {"scale": 1.0},
                           "logit_softcap": 30.0, "norm": {"eps": 1e-6}, "layers": [layer] * n_layers})


def _negunex(width, heads, kv, ff=None, experts=None):
    from llmd_amd.engine.config import negunex_config

    rot = {"dims": 128, "base": 500000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    mixer = {"heads": heads, "kv_heads": kv, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "v_mix": True, "rot": rot}
    mlp = {"kind": "dense", "ff": ff} if ff else \
        {"kind": "moe", "expert": {"ff": experts[2]}, "router": {"experts": experts[0], "identity": 4, "top": experts[1]}}
    return lambda n: negunex_config({"architecture": "Negunex", "width": width, "vocab": 32000, "streams": 2,
                                     "norm": {"eps": 1e-6},
                                     "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp}] * n})


def _zumizen(kind: str):
    from llmd_amd.engine.config import zumizen_config

    if kind == "channel":
        layer = {"type": "channel_delta",
                 "mixer": {"heads": 32, "kv_heads": 32, "dim": 64, "vdim": 64, "conv": 4, "decay_rank": 64,
                           "gate_rank": 64},
                 "mlp": {"kind": "moe", "expert": {"ff": 1408}, "router": {"experts": 64, "top": 6}}}
    else:
        layer = {"type": "parallel",
                 "mixer": {"left": {"heads": 32, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                                    "mask": {"size": 1024}},
                           "right": {"heads": 16, "kv_heads": 8, "dim": 128, "vdim": 128, "conv": 4},
                           "left_scale": 1.0, "right_scale": 1.0},
                 "mlp": {"kind": "moe", "expert": {"ff": 768}, "router": {"experts": 128, "top": 8}}}
    return lambda n: zumizen_config({"architecture": "Zumizen", "name": "zumizen-" + kind, "width": WIDTH,
                                     "vocab": 32000, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
                                     "embedding": {"scale": 1.0,
                                                   "bigram": {"buckets": 65521, "mul_prev": 31337, "mul_cur": 7919}},
                                     "layers": [layer] * n})


def _kakalorn(kind: str):
    from llmd_amd.engine.config import kakalorn_config

    width = 4096 if kind == "window" else WIDTH
    win = {"type": "attention",
           "mixer": {"heads": 32, "kv_heads": 8 if kind == "window" else 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                     "mask": {"size": 1024, "keep_first": 4}, "rot": {"dims": 128, "base": 500000.0}},
           "mlp": {"kind": "dense", "ff": 14336 if kind == "window" else 5632}}
    lat = {"type": "latent_attention",
           "mixer": {"heads": 16, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": 1536,
                     "scale": 192 ** -0.5,
                     "rot": {"dims": 64, "base": 10000.0,
                             "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
           "mlp": {"kind": "dense", "ff": 5632}}
    rec = {"type": "hgrn2", "mixer": {"heads": 32, "dim": 64, "vdim": 64}, "mlp": {"kind": "dense", "ff": 5632}}

    def make(n):
        if kind == "hybrid":
            shared = json.loads(json.dumps(lat))
            layers = []
            for i in range(n):
                layers.append([rec, lat, win, shared][i % 4])
                if i % 4 == 3:
                    layers[-1] = json.loads(json.dumps(shared))
                    layers[-1]["mixer"]["kv_from"] = i - 2
        else:
            layers = [{"window": win, "latent": lat, "hgrn2": rec}[kind]] * n
        return kakalorn_config({"architecture": "Kakalorn", "name": "kakalorn-" + kind, "width": width, "vocab": 32000,
                                "norm": {"eps": 1e-6}, "canon": {"taps": 4}, "layers": layers})

    return make


def _runner(mc, tokens: int, batch: int, device: str):
    from llmd_amd.engine.config import EngineConfig
    from llmd_amd.engine.model_runner import ModelRunner

    bs = 64
    pages = (batch + 1) * (tokens // bs + 2)
    cfg = EngineConfig.create(mc.name, model_config=mc, device=device, block_size=bs, num_gpu_blocks=pages,
                              max_num_seqs=batch + 1, max_model_len=tokens + 65, max_num_batched_tokens=tokens,
                              enforce_eager=True, enable_prefix_caching=False, prefill_token_align=0)
    r = ModelRunner(cfg)
    r.profile_and_allocate()
    return r


def _plans(r, tokens: int, batch: int):
    bs, W = r.bs, r.width
    nb = tokens // bs + 2
    rng = np.random.default_rng(0)
    p_bt = np.zeros((1, W), np.int32)
    p_bt[0, :nb] = np.arange(nb)
    pre = {"graph": False, "nd": 0, "ids": rng.integers(0, 1000, tokens).tolist(), "pos": list(range(tokens)),
           "slots": list(range(tokens)), "d_bt": np.zeros((0, W), np.int32), "d_len": np.zeros(0, np.int32),
           "p_ql": [tokens], "p_ctx": [tokens], "p_bt": p_bt, "rows": [tokens - 1]}
    d_bt = np.zeros((batch, W), np.int32)
    for b in range(batch):
        d_bt[b, :nb] = np.arange(nb) + (b + 1) * nb
    dec = {"graph": False, "nd": batch, "ids": rng.integers(0, 1000, batch).tolist(), "pos": [tokens] * batch,
           "slots": [int(d_bt[b, tokens // bs]) * bs + tokens % bs for b in range(batch)], "d_bt": d_bt,
           "d_len": np.full(batch, tokens + 1, np.int32), "p_ql": [], "p_ctx": [],
           "p_bt": np.zeros((0, W), np.int32), "rows": list(range(batch))}
    if r.seq_steps:
        pre["seq"] = ([0], [0])
        dec["seq"] = (list(range(1, batch + 1)) if r.stateful else [0] * batch, [1] * batch)
    return pre, dec


def _time(r, pl, reps: int) -> float:
    for _ in range(2):
        r.run_plan(pl)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        r.run_plan(pl)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def run(tokens: int = 2048, batch: int = 32, n_layers: int = 4, reps: int = 5, device: str = "cuda",
        only: str = "") -> dict:
    import dataclasses

    from llmd_amd.engine.config import get_model_config

    out = {"tokens": tokens, "batch": batch, "layers": n_layers, "dtype": "bf16", "data": "synthetic", "entries": {}}
    ref = dataclasses.replace(get_model_config("deepseek-v2-lite"), num_hidden_layers=n_layers + 1,
                              first_k_dense_replace=1, vocab_size=32000, rope_scaling=None, name="deepseek-v2-lite-cut")
    todo = [("latent+moe", stack_config(_attn(), n_layers), n_layers), ("mamba", stack_config(_mamba(), n_layers), n_layers),
            ("delta", stack_config(_delta(), n_layers), n_layers), ("deepseek-v2-lite (1 dense + moe layers)", ref, n_layers + 1),
            ("negunex-dense", _negunex(4096, 32, 8, ff=14336)(n_layers), n_layers),
            ("llama-3-8b layers", dataclasses.replace(get_model_config("llama-3-8b"), num_hidden_layers=n_layers,
                                                      vocab_size=32000, name="llama-3-8b-cut"), n_layers),
            ("negunex-moe", _negunex(2048, 32, 4, experts=(128, 8, 768))(n_layers), n_layers),
            ("qwen3-30b-a3b layers", dataclasses.replace(get_model_config("qwen3-30b-a3b"), num_hidden_layers=n_layers,
                                                         vocab_size=32000, name="qwen3-30b-a3b-cut"), n_layers),
            ("zumizen-channel", _zumizen("channel")(n_layers), n_layers),
            ("zumizen-parallel", _zumizen("parallel")(n_layers), n_layers),
            ("kakalorn-window", _kakalorn("window")(n_layers), n_layers),
            ("kakalorn-latent", _kakalorn("latent")(n_layers), n_layers),
            ("kakalorn-hgrn2", _kakalorn("hgrn2")(n_layers), n_layers),
            ("kakalorn-hybrid", _kakalorn("hybrid")(n_layers), n_layers)]
    for name, mc, L in todo:
        if only and not any(name.startswith(o) for o in only.split(",")):
            continue
        r = _runner(mc, tokens, batch, device)
        pre, dec = _plans(r, tokens, batch)
        tp, td = _time(r, pre, reps), _time(r, dec, reps * 4)
        out["entries"][name] = {"prefill_tok_s": round(tokens / tp), "prefill_ms_per_layer": round(tp * 1e3 / L, 3),
                                "decode_tok_s": round(batch / td), "decode_ms_per_layer": round(td * 1e3 / L, 3)}
        del r
        torch.cuda.empty_cache()
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--tokens", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--layers", type=int, default=4)
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--only", default="", help="run the entries whose name starts with one of these (commas between)")
    a = ap.parse_args(argv)
    print(json.dumps(run(a.tokens, a.batch, a.layers, a.reps, only=a.only)), flush=True)


if __name__ == "__main__":
    main()
