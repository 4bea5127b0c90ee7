"""A model described as data: which parts each layer is made of, and in
which order the layers run.

Nothing here knows an architecture.  An architecture (see ``registry.py``)
turns its typed configuration into a :class:`ModelLayout`; the model
builder turns the layout into parts by looking each ``PartSpec.kind`` up
in the part registries of ``fastgen_amd.parts``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: its kind, the tensor-name prefix under which its
    weights are stored, and its sizes and constants."""

    kind: str
    prefix: str = ""
    options: Mapping[str, Any] = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.options.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a token mixer and a feed-forward, each with its norm, and
    the name of the arrangement that wires them to the residual stream.
    ``extra_norms``: further norms by name, for arrangements that own more
    than two (norms after the mixer and the feed-forward, say); the
    arrangement gets them as a dict."""

    mixer: PartSpec
    ffn: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec
    arrangement: str = "pre_norm"
    extra_norms: Mapping[str, PartSpec] = field(default_factory=dict)


@dataclass(frozen=True)
class RunEntry:
    """One item of the execution order.

    ``layer`` indexes ``ModelLayout.layers``; the same layer may be named
    by several entries.  Every entry owns storage of its own (pages or a
    state slot) unless ``reads_cache_of`` names an earlier entry of the
    order: then its mixer writes nothing and reads that entry's storage.
    """

    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelLayout:
    dim: int
    vocab_size: int
    embed: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec

    def __post_init__(self) -> None:
        for i, e in enumerate(self.order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"order[{i}] names layer {e.layer}, which does not exist")
            if e.reads_cache_of is not None:
                j = e.reads_cache_of
                if not 0 <= j < i:
                    raise ValueError(
                        f"order[{i}] reads the cache of order[{j}], which does not run before it"
                    )
                if self.order[j].reads_cache_of is not None:
                    raise ValueError(
                        f"order[{i}] reads the cache of order[{j}], which owns none"
                    )
