"""The description of a model as data: parts, layers, and the order they run in.

An architecture's builder turns its typed configuration into a ``ModelSpec``.
Nothing below the builder knows which architecture it serves: every part gets
its sizes and constants from its ``PartSpec`` and finds its tensors under the
name prefix it is given.

The reference keeps the same facts as per-layer arrays on its model record:
which layers are windowed, which layer owns the cache rows a layer reads
(``model_kv_owner``), per-layer head counts and rotary widths
(src/model.h:423-510).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: the registered ``kind`` and the parameters its constructor takes."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    prefix: str = ""        # the part's tensors are stored as prefix + relative name

    def __hash__(self):
        return hash((self.kind, self.prefix, repr(sorted(self.params.items(), key=lambda kv: kv[0]))))


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts.

    ``block`` names the arrangement (how norms, mixer, feed-forward and the residual sums
    follow each other); ``norms`` holds the norms that arrangement has, under the names it
    gives them ("prenorm": ``mixer_norm`` and ``feed_forward_norm``; an arrangement with a
    third norm simply names three).  An arrangement may do without a mixer or without a
    feed-forward.
    """
    mixer: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    norms: Mapping[str, PartSpec] = field(default_factory=dict)
    block: str = "prenorm"


@dataclass(frozen=True)
class ExecStep:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named by several
    entries: its weights are shared, each entry has a cache of its own).
    ``cache_of`` is the index of an earlier entry whose cache this entry reads
    instead of owning one; such an entry writes no keys or values.
    """
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: PartSpec
    layers: List[LayerSpec]
    order: List[ExecStep]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None

    def validate(self) -> None:
        for i, st in enumerate(self.order):
            if not (0 <= st.layer < len(self.layers)):
                raise ValueError(f"run order entry {i} names layer {st.layer}, model has {len(self.layers)}")
            if st.cache_of is not None:
                if not (0 <= st.cache_of < i):
                    raise ValueError(f"run order entry {i} reads the cache of entry {st.cache_of}, "
                                     f"which does not run before it")
                if self.order[st.cache_of].cache_of is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {st.cache_of}, "
                                     f"which owns none")
