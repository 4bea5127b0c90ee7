"""What a part is, and the registries that map a ``PartSpec.kind`` to one.

A part is built from a :class:`~fastgen_amd.config.PartSpec` alone: its
sizes and constants are the spec's options, its tensors are named by the
spec's prefix.  No part knows which model it sits in.  Five kinds of part
have a registry each (mixer, feed-forward, norm, position encoding, block
arrangement) next to the two ends of the model (embedding, head).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping, Optional, Sequence, Tuple

import torch

from ..config.layout import PartSpec

# ---------------------------------------------------------------- tensors
MATRIX = "matrix"  # operand of a matrix product, or a table of rows: compute dtype
VECTOR = "vector"  # per-channel constants: stay fp32 when stored so
TABLE_INT = "int"  # integer tables: int32


@dataclass(frozen=True)
class TensorSpec:
    name: str  # full name in the checkpoint
    shape: Tuple[int, ...]
    role: str = MATRIX
    # how random weights for it are drawn: ("normal", std) or ("one_plus_normal", std)
    init: Tuple[str, float] = ("normal", 0.02)


def place(t: torch.Tensor, role: str, dtype: torch.dtype, device: torch.device | str) -> torch.Tensor:
    """Move a loaded tensor to the device in the dtype the engine keeps it in.

    Matrices and row tables take the compute dtype (bfloat16, or float32 on
    the 32-bit path); integer tables become int32; a vector stored in 32-bit
    stays 32-bit, because the kernels that use it compute in fp32 anyway.
    """
    if not t.dtype.is_floating_point:
        return t.to(device=device, dtype=torch.int32).contiguous()
    if role == VECTOR and t.dtype == torch.float32:
        return t.to(device=device).contiguous()
    return t.to(device=device, dtype=dtype).contiguous()


# ------------------------------------------------------------------ needs
@dataclass(frozen=True)
class PagedNeed:
    """Per-token storage: keys and values of ``n_kv_heads`` heads of
    ``head_dim``; with ``window`` only the last ``window`` tokens are read.
    ``v_head_dim``: the width of a value where it differs from a key's (the
    built-in attention kernels take equal widths only; a mixer with a cache of
    two widths reads and writes its pages itself)."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None

    @property
    def value_dim(self) -> int:
        return self.v_head_dim or self.head_dim


@dataclass(frozen=True)
class StateNeed:
    """Per-request storage of fixed size, zero when a request is admitted."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerStore:
    """The storage handed to a mixer for one entry of the run order."""

    group: Optional[int] = None  # index of its cache group in StepContext.groups
    k_pages: Optional[torch.Tensor] = None  # [n_pages, KV, P, hd]
    v_pages: Optional[torch.Tensor] = None  # [n_pages, KV, hd, P] (hd: the need's value_dim)
    state: Optional[torch.Tensor] = None  # [n_slots, *StateNeed.shape]
    owns: bool = True  # False: the storage belongs to an earlier entry; read only


class Part:
    """Base of every part: declares its tensors and takes them when loaded.

    ``capturable``: whether ``forward`` may be recorded into a HIP graph, that
    is, whether it launches the same kernels with the same arguments whatever
    the values on the device are, and takes everything that changes from step
    to step (tokens, positions, lengths, block tables, slot ids) from the
    context's device tensors.  A part that looks at device data on the host
    (shapes that depend on the data), or that uses the context's host copies
    in a step of one token a sequence, sets it to False; a model with such a
    part is always stepped eagerly.  Only steps in which every sequence brings
    one token are recorded; a recorded step may hold stand-in sequences, whose
    state slot (``ctx.slot_ids``) is a row that belongs to no request."""

    capturable: bool = True

    def __init__(self, spec: PartSpec) -> None:
        self.spec = spec
        self.prefix = spec.prefix

    def _name(self, suffix: str) -> str:
        return f"{self.prefix}.{suffix}" if self.prefix else suffix

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        pass


class Mixer(Part):
    """A token mixer: rows in, rows out, with storage per token or per request.

    ``forward(x, ctx, store)`` gets the normed rows ``[T, dim]`` of the step,
    the step's ragged description and its storage, and returns ``[T, dim]``
    rows in the same dtype to be added to the residual stream (or fp32
    ``[S, T, dim]`` partial sums whose sum is that; the norm adds them).  What
    one step writes to the storage is what the next step of the same request
    reads.
    """

    def paged_need(self) -> Optional[PagedNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, ctx: Any, store: LayerStore) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Rows in, rows out; no storage, indifferent to the ragged batch."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    """A norm on the fp32 residual stream, fused with the addition before it.

    ``forward(h, delta, rows=None)`` adds ``delta`` (or nothing) to ``h`` in
    place and returns the normed rows in ``dtype``; with ``rows`` only those
    rows are returned and ``h`` is left as it was.  ``delta`` is ``[T, dim]`` in
    ``dtype`` or fp32 ``[S, T, dim]`` partial sums to be added in order.
    """

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer.  A rotary scheme gives a frequency table,
    the number of leading head dimensions it rotates, and the row order in
    which the q/k projection weights must be stored for its pairing."""

    rotary_dim: int = 0

    def frequencies(self) -> Optional[torch.Tensor]:
        return None

    def frequencies_on(self, device: Any) -> Optional[torch.Tensor]:
        """The frequency table on ``device``; parts with equal tables share one
        tensor, so that what is derived from it per step is computed once."""
        f = self.frequencies()
        if f is None:
            return None
        key = (str(torch.device(device)), tuple(f.tolist()))
        if key not in _FREQUENCY_TABLES:
            _FREQUENCY_TABLES[key] = f.to(device=device, dtype=torch.float32).contiguous()
        return _FREQUENCY_TABLES[key]

    def arrange_rows(self, w: torch.Tensor, n_heads: int) -> torch.Tensor:
        return w


_FREQUENCY_TABLES: Dict[Tuple[str, Tuple[float, ...]], torch.Tensor] = {}


# -------------------------------------------------------------- registries
_REGISTRIES: Dict[str, Dict[str, Callable[[PartSpec], Any]]] = {
    "mixer": {},
    "feed_forward": {},
    "norm": {},
    "position": {},
    "arrangement": {},
    "embedding": {},
    "head": {},
}


def register_part(category: str, kind: str, factory: Callable[..., Any], *, replace: bool = False) -> None:
    reg = _REGISTRIES[category]
    if kind in reg and not replace:
        raise ValueError(f"{category} {kind!r} is already registered")
    reg[kind] = factory


def unregister_part(category: str, kind: str) -> None:
    _REGISTRIES[category].pop(kind, None)


def build_part(category: str, spec: PartSpec, *args: Any) -> Any:
    reg = _REGISTRIES[category]
    if spec.kind not in reg:
        raise KeyError(f"no {category} of kind {spec.kind!r}; registered: {sorted(reg)}")
    return reg[spec.kind](spec, *args)


def registered_parts(category: str) -> Sequence[str]:
    return sorted(_REGISTRIES[category])
