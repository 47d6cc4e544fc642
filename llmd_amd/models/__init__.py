"""Model registry: HF ``model_type`` -> implementation."""
from __future__ import annotations

import torch

from llmd_amd.engine.config import ModelConfig


def model_class(cfg: ModelConfig):
    t = cfg.model_type
    if t in ("llama", "qwen3", "qwen2", "mistral"):
        from .llama import LlamaForCausalLM

        return LlamaForCausalLM
    if t == "opt":
        from .opt import OPTForCausalLM

        return OPTForCausalLM
    if t == "llava":
        from .vision import LlavaForCausalLM

        return LlavaForCausalLM
    if t == "gpt_oss":
        from .gpt_oss import GptOssForCausalLM

        return GptOssForCausalLM
    if t in ("deepseek", "deepseek_v3", "deepseek_v2"):
        from .deepseek import DeepseekForCausalLM

        return DeepseekForCausalLM
    if t in ("mixtral", "qwen3_moe"):
        from .moe_llama import MoELlamaForCausalLM

        return MoELlamaForCausalLM
    if t == "mekusun":
        from .mekusun import MekusunForCausalLM

        return MekusunForCausalLM
    if t == "negunex":
        from .negunex import NegunexForCausalLM

        return NegunexForCausalLM
    if t == "zumizen":
        from .zumizen import ZumizenForCausalLM

        return ZumizenForCausalLM
    if t == "kakalorn":
        from .kakalorn import KakalornForCausalLM

        return KakalornForCausalLM
    raise ValueError(f"unsupported model_type {t!r}")


def build_model(cfg: ModelConfig, device="cuda", max_pos: int = 32768, dtype=None):
    cls = model_class(cfg)
    if dtype is not None and dtype != torch.bfloat16:
        if not getattr(cls, "supports_float32", False):
            raise ValueError(f"{cfg.model_type} runs in bfloat16 only")
        return cls(cfg, device=device, max_pos=max_pos, dtype=dtype)
    return cls(cfg, device=device, max_pos=max_pos)
