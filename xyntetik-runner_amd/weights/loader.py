"""Binding a model's tensors by name, with one error that tells everything wrong.

The reference looks every tensor up by name, refuses the load when one is missing
(``need_tensor``, src/model.c:158-170) and checks each shape
against the geometry with a message that names tensor, layer, got and expected
(``check_shape``, src/model.c:193-205).  Here all findings of one
load are gathered: missing tensors, tensors the model has no use for, and wrong
shapes or dtypes come in a single ``WeightError``.

dtype rule: in a bfloat16 engine a "matrix" is kept in bfloat16; a "vector" stored
in 32 bits stays so; integer tables become int32.  In a float32 engine everything
floating is widened to float32, which is exact for bfloat16 and float16.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Mapping, Optional, Tuple

import torch

from ..parts.base import ParamSpec
from .safetensors_io import SafetensorsStore

_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int32, torch.int64)
# buffers some exporters write that are no parameters
IGNORED_SUFFIXES = ("rotary_emb.inv_freq",)


class WeightError(ValueError):
    def __init__(self, missing: List[str], unexpected: List[str], wrong: List[str]):
        self.missing, self.unexpected, self.wrong = missing, unexpected, wrong
        lines = ["the checkpoint does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape or dtype ({len(wrong)}):")
            lines.extend("    " + w for w in wrong)
        super().__init__("\n".join(lines))


def target_dtype(spec: ParamSpec, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if spec.role == "int":
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if spec.role == "vector":
        return torch.bfloat16 if stored == torch.bfloat16 else torch.float32
    return compute


def check_against(expected: Mapping[str, ParamSpec], names: Iterable[str],
                  shape_of: Callable[[str], Tuple[int, ...]],
                  dtype_of: Callable[[str], torch.dtype]) -> None:
    """Raise ``WeightError`` unless the stored tensors are exactly what the model expects."""
    names = list(names)
    have = set(names)
    missing = [n for n, s in expected.items() if n not in have and not s.optional]
    unexpected = sorted(n for n in have if n not in expected and not n.endswith(IGNORED_SUFFIXES))
    wrong = []
    for n, s in expected.items():
        if n not in have:
            continue
        shp, dt = tuple(shape_of(n)), dtype_of(n)
        if shp != tuple(s.shape):
            wrong.append(f"{n}: stored {list(shp)}, the model needs {list(s.shape)}")
        elif s.role == "int" and dt not in _INTS:
            wrong.append(f"{n}: stored as {dt}, the model needs an integer table")
        elif s.role != "int" and dt not in _FLOATS:
            wrong.append(f"{n}: stored as {dt}, the model needs a floating-point tensor")
    if missing or unexpected or wrong:
        raise WeightError(sorted(missing), unexpected, wrong)


def load_tensors(store: SafetensorsStore, expected: Mapping[str, ParamSpec], compute: torch.dtype,
                 device: torch.device) -> Dict[str, torch.Tensor]:
    """All expected tensors present in ``store``, on ``device``, in the dtype their role asks for."""
    check_against(expected, store.names(), store.shape, store.dtype)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        if name not in store:
            continue
        t = store.tensor(name)
        dt = target_dtype(spec, t.dtype, compute)
        # widen or narrow on the host only when the device cannot take the stored type as it is
        if t.dtype in (torch.float16, torch.float64) or (t.dtype == torch.int64):
            t = t.to(dt)
        out[name] = t.to(device=device, dtype=dt, non_blocking=False).contiguous()
    return out


def load_state(tensors: Mapping[str, torch.Tensor], expected: Mapping[str, ParamSpec], compute: torch.dtype,
               device: torch.device, consume: bool = False) -> Dict[str, torch.Tensor]:
    """As ``load_tensors`` for tensors already in memory (the random-weights mode without a file).
    With ``consume`` the tensors are taken out of ``tensors`` (a dict) as they are used, so that a
    model as large as half the memory does not stand there twice."""
    check_against(expected, tensors.keys(), lambda n: tuple(tensors[n].shape), lambda n: tensors[n].dtype)
    out = {}
    for name, spec in expected.items():
        if name in tensors:
            t = tensors.pop(name) if consume else tensors[name]
            out[name] = t.to(device=device, dtype=target_dtype(spec, t.dtype, compute)).contiguous()
    return out
