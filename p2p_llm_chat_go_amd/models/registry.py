"""Model registry: which config, weight store and engine serve a checkpoint or preset.

A checkpoint folder is recognised by its ``config.json``: an ``architecture`` key naming a
hybrid design (``models.hybrid.DESIGNS``) selects ``models.hybrid`` + ``engine.hybrid``;
anything else is read as an HF Llama / Mixtral config (``models.weights``) for ``Engine``.
"""
from __future__ import annotations

import json
import os

import torch

def hybrid_architectures() -> tuple:
    from .hybrid import DESIGNS

    return tuple(DESIGNS)


def is_hybrid_dir(path: str) -> bool:
    with open(os.path.join(path, "config.json")) as f:
        return json.load(f).get("architecture") in hybrid_architectures()


def supports_dtype(path: str, dtype) -> bool:
    """Hybrid models run in bfloat16 or float32; the Llama / Mixtral kernels are bf16 only."""
    return dtype == torch.bfloat16 or is_hybrid_dir(path)


def load_checkpoint(path: str, device="cuda", dtype=torch.bfloat16):
    """(config, weights) of a checkpoint folder, by its config.json."""
    if is_hybrid_dir(path):
        from .hybrid import load_dir

        return load_dir(path, device, dtype)
    if dtype != torch.bfloat16:
        raise ValueError("Llama / Mixtral checkpoints are served in bfloat16 only")
    from .weights import EngineWeights, config_from_hf, load_safetensors_dir

    cfg = config_from_hf(path)
    return cfg, EngineWeights.from_state_dict(load_safetensors_dir(path, device), cfg, device)


def make_engine(cfg, weights=None, device="cuda", **kw):
    """The engine class that serves this config."""
    from .hybrid import HybridConfig

    if isinstance(cfg, HybridConfig):
        from ..engine.hybrid import HybridEngine

        return HybridEngine(cfg, weights=weights, device=device, **kw)
    from ..engine import Engine

    kw.pop("dtype", None)
    kw.pop("num_slots", None)
    return Engine(cfg, weights=weights, device=device, **kw)
