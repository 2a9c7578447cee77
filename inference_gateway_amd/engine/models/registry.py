"""Model registry: which class serves which architecture, and how a
checkpoint directory's config.json maps to an engine model config."""
from __future__ import annotations

import json
import struct
from pathlib import Path

import torch

from ..config import (BozolornConfig, FedatarConfig, FeditarConfig,
                      MekevikConfig, ModelConfig)


def build_model(model_cfg, device, dtype):
    """Instantiate the model class for a config object."""
    if isinstance(model_cfg, FedatarConfig):
        from .fedatar import FedatarForCausalLM as cls
    elif isinstance(model_cfg, MekevikConfig):
        from .mekevik import MekevikForCausalLM as cls
    elif isinstance(model_cfg, FeditarConfig):
        from .feditar import FeditarForCausalLM as cls
    elif isinstance(model_cfg, BozolornConfig):
        from .bozolorn import BozolornForCausalLM as cls
    elif model_cfg.is_moe:
        from .mixtral import MixtralForCausalLM as cls
    else:
        from .llama import LlamaForCausalLM as cls
    supported = getattr(cls, "supported_dtypes", (torch.bfloat16,))
    if dtype not in supported and torch.device(device).type == "cuda":
        raise ValueError(
            f"{cls.__name__} has no {dtype} kernels on the GPU "
            f"(supported: {supported})")
    return cls(model_cfg, device, dtype)


def safetensors_shapes(path: str) -> dict:
    """Tensor name -> shape from the headers of a directory's
    *.safetensors files (8-byte little-endian length, then JSON);
    reads no tensor data."""
    shapes = {}
    for f in sorted(Path(path).glob("*.safetensors")):
        with open(f, "rb") as fh:
            (n,) = struct.unpack("<Q", fh.read(8))
            header = json.loads(fh.read(n))
        for name, meta in header.items():
            if name != "__metadata__":
                shapes[name] = list(meta["shape"])
    return shapes


def model_config_from_dir(path: str):
    """Pick the architecture by the directory's config.json: the
    per-layer designs name themselves with an `architecture` key;
    everything else is read as a HuggingFace Llama-family config."""
    cfg = json.loads((Path(path) / "config.json").read_text())
    if cfg.get("architecture") == "Mekevik":
        return MekevikConfig.from_dict(
            cfg, name=Path(path).name or "mekevik",
            shapes=safetensors_shapes(path))
    if cfg.get("architecture") == "Feditar":
        return FeditarConfig.from_dict(
            cfg, name=Path(path).name or "feditar",
            shapes=safetensors_shapes(path))
    if cfg.get("architecture") == "Bozolorn":
        return BozolornConfig.from_dict(
            cfg, name=Path(path).name or "bozolorn",
            shapes=safetensors_shapes(path))
    if cfg.get("architecture") == "Fedatar":
        return FedatarConfig.from_dict(
            cfg, name=Path(path).name or "fedatar",
            shapes=safetensors_shapes(path))
    from ..weights import model_config_from_hf

    return model_config_from_hf(path)


def is_recurrent(model_cfg) -> bool:
    """True when some layer keeps per-sequence state outside the paged
    cache (prefix reuse across requests is then impossible: the state at
    a shared prefix's end is not stored)."""
    if isinstance(model_cfg, FeditarConfig):
        return True     # every mixer and the embedding keep slot state
    if isinstance(model_cfg, BozolornConfig):
        # the delta-rule half of a parallel mixer keeps slot state
        return any(l.type == "parallel" for l in model_cfg.layers)
    return isinstance(model_cfg, FedatarConfig) and any(
        l.type == "mingru" for l in model_cfg.layers)


__all__ = ["build_model", "model_config_from_dir", "safetensors_shapes",
           "is_recurrent", "ModelConfig", "FedatarConfig", "MekevikConfig",
           "FeditarConfig", "BozolornConfig"]
