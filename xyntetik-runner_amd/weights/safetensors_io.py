"""Reading and writing safetensors files, by tensor name.

File layout: an 8-byte little-endian header length ``n``, ``n`` bytes of JSON
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}``
and the tensor bytes, offsets counted from the end of the header.

The checks are those the reference makes on its own container: every tensor's
byte range lies inside the mapping and is overflow-checked
(src/gguf.c:229-280), names are unique (:191-215), and a lookup is
by exact name (:579-583).  The file is memory-mapped; a tensor's bytes are touched
only when it is asked for.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import torch

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
    "F64": (torch.float64, 8),
    "U8": (torch.uint8, 1),
    "I8": (torch.int8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
MAX_HEADER = 100 * 1024 * 1024


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int          # absolute byte offset in the file
    nbytes: int
    file: int           # index into SafetensorsStore.files


def _no_duplicates(pairs):
    seen = {}
    for k, v in pairs:
        if k in seen:
            raise SafetensorsError(f"tensor name {k!r} appears twice in the header")
        seen[k] = v
    return seen


class _MappedFile:
    def __init__(self, path: str):
        self.path = path
        self.size = os.path.getsize(path)
        if self.size < 8:
            raise SafetensorsError(f"{path}: {self.size} bytes is too short for a safetensors file")
        self._fh = open(path, "rb")
        self.map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self.map[:8])
        if hlen > MAX_HEADER or 8 + hlen > self.size:
            raise SafetensorsError(
                f"{path}: header length {hlen} does not fit the file ({self.size} bytes); truncated or not safetensors")
        try:
            self.header = json.loads(self.map[8:8 + hlen].decode("utf-8"), object_pairs_hook=_no_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        if not isinstance(self.header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.data_start = 8 + hlen

    def close(self):
        try:
            self.map.close()
        except BufferError:
            pass        # tensors made from the mapping are still alive
        self._fh.close()


class SafetensorsStore:
    """All tensors of a model folder (one file, or shards named by an index)."""

    def __init__(self, paths: Iterable[str]):
        self.files: List[_MappedFile] = []
        self.entries: Dict[str, TensorEntry] = {}
        for path in paths:
            mf = _MappedFile(path)
            fi = len(self.files)
            self.files.append(mf)
            for name, info in mf.header.items():
                if name == "__metadata__":
                    continue
                if name in self.entries:
                    raise SafetensorsError(f"{path}: tensor {name!r} is also in {self.files[self.entries[name].file].path}")
                self.entries[name] = self._entry(mf, fi, name, info)

    @staticmethod
    def _entry(mf: _MappedFile, fi: int, name: str, info) -> TensorEntry:
        try:
            dtype = info["dtype"]
            shape = tuple(int(s) for s in info["shape"])
            begin, end = (int(o) for o in info["data_offsets"])
        except (KeyError, TypeError, ValueError):
            raise SafetensorsError(f"{mf.path}: malformed header entry for {name!r}") from None
        if dtype not in _DTYPES:
            raise SafetensorsError(f"{mf.path}: tensor {name!r} has unsupported dtype {dtype!r}")
        if any(s < 0 for s in shape):
            raise SafetensorsError(f"{mf.path}: tensor {name!r} has a negative dimension {shape}")
        numel = 1
        for s in shape:
            numel *= s
        nbytes = numel * _DTYPES[dtype][1]
        if begin < 0 or end < begin or end - begin != nbytes:
            raise SafetensorsError(
                f"{mf.path}: tensor {name!r} {dtype}{list(shape)} needs {nbytes} bytes, offsets give {end - begin}")
        if mf.data_start + end > mf.size:
            raise SafetensorsError(
                f"{mf.path}: tensor {name!r} ends at byte {mf.data_start + end}, file has {mf.size} (truncated?)")
        return TensorEntry(name, dtype, shape, mf.data_start + begin, nbytes, fi)

    @staticmethod
    def open_folder(model_dir: str) -> "SafetensorsStore":
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        if os.path.exists(index):
            with open(index, "r", encoding="utf-8") as f:
                wm = json.load(f).get("weight_map", {})
            shards = sorted(set(wm.values()))
            if not shards:
                raise SafetensorsError(f"{index}: empty weight_map")
            return SafetensorsStore(os.path.join(model_dir, s) for s in shards)
        if os.path.exists(single):
            return SafetensorsStore([single])
        raise SafetensorsError(f"{model_dir}: no model.safetensors (or model.safetensors.index.json)")

    def names(self) -> List[str]:
        return list(self.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name].shape

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name].dtype][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor over the mapped bytes (read-only memory: copy before writing)."""
        e = self.entries[name]
        dt = _DTYPES[e.dtype][0]
        if e.nbytes == 0:
            return torch.empty(e.shape, dtype=dt)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # torch warns that the buffer is not writable
            flat = torch.frombuffer(self.files[e.file].map, dtype=torch.uint8, count=e.nbytes, offset=e.begin)
        return flat.view(dt).reshape(e.shape)

    def close(self):
        for mf in self.files:
            mf.close()


def save_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                     metadata: Optional[Mapping[str, str]] = None) -> None:
    """Write ``tensors`` (CPU, contiguous or not) to ``path``; names in sorted order."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store tensor {name!r} of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
