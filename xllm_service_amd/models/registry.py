"""Model factory."""
from __future__ import annotations

import torch

from .config import ModelConfig


def create_model(cfg: ModelConfig, dtype=torch.bfloat16):
    if cfg.architecture == "llama":
        from .llama import LlamaForCausalLM
        return LlamaForCausalLM(cfg, dtype=dtype)
    if cfg.architecture == "opt":
        from .opt import OPTForCausalLM
        return OPTForCausalLM(cfg, dtype=dtype)
    if cfg.architecture in ("qwen2", "qwen2_vl"):
        # plain Qwen2 text models share the VL language tower exactly
        # (llama stack + qkv bias); the vision tower is a separate class
        from .qwen2_vl import Qwen2VLForCausalLM
        return Qwen2VLForCausalLM(cfg, dtype=dtype)
    if cfg.architecture == "pugovik":
        from .pugovik import PugovikForCausalLM
        return PugovikForCausalLM(cfg, dtype=dtype)
    if cfg.architecture == "dunusun":
        from .dunusun import DunusunForCausalLM
        return DunusunForCausalLM(cfg, dtype=dtype)
    if cfg.architecture == "tosipel":
        from .tosipel import TosipelForCausalLM
        return TosipelForCausalLM(cfg, dtype=dtype)
    if cfg.architecture == "gararax":
        from .gararax import GararaxForCausalLM
        return GararaxForCausalLM(cfg, dtype=dtype)
    raise ValueError(f"unknown architecture {cfg.architecture}")


def required_extensions(cfg: ModelConfig):
    """In-tree HIP extension modules the model's GPU path loads."""
    if cfg.architecture in ("pugovik", "dunusun", "tosipel", "gararax"):
        return ["_ops_hybrid"]
    return ["_ops"]
