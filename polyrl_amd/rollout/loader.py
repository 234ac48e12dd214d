"""Build a rollout engine from a checkpoint folder (config.json +
*.safetensors): the config's architecture picks the model family, tensor
shapes fill the sizes the config leaves open, and weights load by name."""
from __future__ import annotations

import glob
import json
import os
import struct
from typing import Dict

import torch


def safetensors_shapes(path: str) -> Dict[str, tuple]:
    """name -> shape from a safetensors header (no tensor data is read)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in head.items()
            if k != "__metadata__"}


def engine_from_dir(path: str, device: str = "cuda",
                    dtype: torch.dtype = torch.bfloat16, **engine_kw):
    from safetensors.torch import load_file

    from ..models.registry import get_model_config
    from .engine import Engine
    cfg = get_model_config(path)
    files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors under {path}")
    if getattr(cfg, "is_hybrid", False):
        from .hybrid_model import HybridInferenceModel
        shapes: Dict[str, tuple] = {}
        for f in files:
            shapes.update(safetensors_shapes(f))
        HybridInferenceModel.resolve_shapes(cfg, shapes)
    engine = Engine(cfg, device=device, dtype=dtype, **engine_kw)
    sd = {}
    for f in files:
        sd.update(load_file(f))
    engine.model.load_state_dict(sd, strict=True)
    return engine
