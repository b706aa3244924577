"""Model class by configuration: the engine builds every model through :func:`build_model`."""
from __future__ import annotations

from typing import Optional

import torch

from ..parallel.comm import SINGLE, ParallelContext
from .configs import HybridConfig, ModelConfig


def model_class(cfg):
    if isinstance(cfg, HybridConfig):
        from .hybrid import HybridModel
        return HybridModel
    if isinstance(cfg, ModelConfig):
        from .llama import LlamaModel
        return LlamaModel
    raise TypeError(f"no model class for {type(cfg).__name__}")


def build_model(cfg, device="cuda", dtype=torch.bfloat16, par: ParallelContext = SINGLE, seed: int = 0,
                weights: Optional[str] = None):
    return model_class(cfg)(cfg, device=device, dtype=dtype, par=par, seed=seed, weights=weights)
