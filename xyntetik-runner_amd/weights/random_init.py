"""The random-weights mode: a model folder from a configuration and a seed.

Every tensor has a generator of its own, seeded from (seed, tensor name), so a
tensor's values do not depend on which other tensors exist or in which order they
are made.  Matrices are N(0, std) (std 0.02 unless told otherwise) rounded to the
storage dtype; norm weights are 1, or 1 + N(0, jitter).  The reference's fixture
generator plays the same role with an LCG and weights uniform in +-0.04, norm
weights 1.0 (scripts/make-test-model.py:238-252).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Mapping, Optional

import torch

from ..parts.base import ParamSpec
from .safetensors_io import save_safetensors

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec: ParamSpec, seed: int, std: float, jitter: float,
                  matrix_dtype: torch.dtype, vector_dtype: torch.dtype,
                  device: Optional[torch.device] = None) -> torch.Tensor:
    dev = device or torch.device("cpu")
    g = torch.Generator(device=dev)
    g.manual_seed(tensor_seed(seed, name))
    dt = torch.int32 if spec.role == "int" else (vector_dtype if spec.role == "vector" else matrix_dtype)
    if spec.init == "normal":
        t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=dev) * std
    elif spec.init == "ones":
        t = torch.ones(spec.shape, dtype=torch.float32, device=dev)
    elif spec.init == "ones_jitter":
        t = torch.ones(spec.shape, dtype=torch.float32, device=dev)
        if jitter:
            t = t + torch.randn(spec.shape, generator=g, dtype=torch.float32, device=dev) * jitter
    elif spec.init == "zeros":
        t = torch.zeros(spec.shape, dtype=torch.float32, device=dev)
    else:
        raise ValueError(f"tensor {name}: unknown init {spec.init!r}")
    return t.to(dt)


def random_state(expected: Mapping[str, ParamSpec], seed: int, std: float = 0.02, jitter: float = 0.0,
                 dtype: str = "bfloat16", vector_dtype: Optional[str] = None,
                 device: Optional[torch.device] = None, include_optional: bool = True) -> Dict[str, torch.Tensor]:
    md = _STORAGE[dtype]
    vd = _STORAGE[vector_dtype] if vector_dtype else md
    return {name: random_tensor(name, spec, seed, std, jitter, md, vd, device)
            for name, spec in expected.items() if include_optional or not spec.optional}


def write_random_model(config: Mapping[str, Any], out_dir: str, seed: int, std: float = 0.02,
                       norm_jitter: float = 0.0, dtype: str = "bfloat16",
                       vector_dtype: Optional[str] = None, device: Optional[torch.device] = None) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors`` for ``config`` (a config.json dict).
    ``device``: where the values are drawn (a large model is drawn much faster on the GPU; the
    values depend on the device's generator, the file is what counts)."""
    from ..config import config_from_dict
    from ..engine.model import Model
    arch, typed = config_from_dict(config)
    spec = arch.build_spec(typed)
    expected = Model.expected_tensors(spec)
    state = random_state(expected, seed, std=std, jitter=norm_jitter, dtype=dtype, vector_dtype=vector_dtype,
                         device=torch.device(device) if device is not None else None)
    os.makedirs(out_dir, exist_ok=True)
    cfg = dict(config)
    cfg.setdefault("torch_dtype", dtype)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    save_safetensors(os.path.join(out_dir, "model.safetensors"), state,
                     metadata={"format": "pt", "seed": str(seed)})
    return out_dir
