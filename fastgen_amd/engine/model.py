"""A model: parts built from a layout, loaded from a tensor source, and run
entry by entry of the layout's order.

The reference's counterpart is the weight-only ``Transformer`` skeleton
(``fastgen/model.py:151-202``) plus the layer loop of ``_forward``
(``fastgen/forward.py:347-515``).
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, List, Mapping, Optional, Sequence

import torch

from ..config import ModelLayout, PartSpec, get_architecture, read_config_json
from ..kernels.linear import StreamedMatrix, packing, packing_fits
from ..kernels.ops import ScaledRows
from ..parts import LayerStore, PagedNeed, StateNeed, TensorSpec, build_part
from ..parts.base import MATRIX
from ..weights.source import RandomSource, SafetensorsSource, TensorSource, check_against_specs
from .context import StepContext


@dataclass
class ModelParts:
    layout: ModelLayout
    embed: Any
    blocks: List[Any]
    mixers: List[Any]
    final_norm: Any
    head: Any
    all_parts: List[Any]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self.all_parts for s in p.tensor_specs()]

    def duplicates(self) -> Mapping[str, str]:
        return dict(self.head.duplicates()) if hasattr(self.head, "duplicates") else {}


def build_parts(layout: ModelLayout) -> ModelParts:
    """Every part of the layout, looked up by kind; nothing is on a device yet."""
    embed = build_part("embedding", layout.embed)
    blocks, mixers, parts = [], [], [embed]
    for ls in layout.layers:
        mixer = build_part("mixer", ls.mixer)
        ffn = build_part("feed_forward", ls.ffn)
        n1 = build_part("norm", ls.mixer_norm)
        n2 = build_part("norm", ls.ffn_norm)
        extra = {name: build_part("norm", spec) for name, spec in ls.extra_norms.items()}
        # an arrangement that asks for no further norms is built from the four parts alone
        blocks.append(build_part("arrangement", PartSpec(ls.arrangement), mixer, ffn, n1, n2, *([extra] if extra else [])))
        mixers.append(mixer)
        parts += [mixer, ffn, n1, n2, *extra.values()]
    final_norm = build_part("norm", layout.final_norm)
    head = build_part("head", layout.head)
    parts += [final_norm, head]
    return ModelParts(layout, embed, blocks, mixers, final_norm, head, parts)


class Model:
    def __init__(self, layout: ModelLayout, dtype: torch.dtype, device: torch.device | str, args: Any = None,
                 architecture: Optional[str] = None, packed_weights: Optional[bool] = None,
                 memory_budget: Optional[int] = None) -> None:
        """``packed_weights``: whether the bfloat16 matrices get a second copy in the order in which the
        products of few rows read them (``kernels.linear.StreamedMatrix``); None: if the weights twice
        leave half of ``memory_budget`` (bytes for the model and its cache; default: the GPU's memory) free
        (``kernels.linear.packing_fits``)."""
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype {dtype} is not supported (float32 or bfloat16)")
        self.layout, self.dtype, self.device = layout, dtype, torch.device(device)
        self.args, self.architecture = args, architecture
        self.packed_weights, self.memory_budget = packed_weights, memory_budget
        self.parts = build_parts(layout)
        self.vocab_size = layout.vocab_size
        self.loaded = False

    # ------------------------------------------------------------- build
    @classmethod
    def from_config(cls, config: Mapping[str, Any], dtype: torch.dtype, device: torch.device | str,
                    packed_weights: Optional[bool] = None, memory_budget: Optional[int] = None) -> "Model":
        arch = get_architecture(config)
        args = arch.parse(config)
        return cls(arch.layout(args), dtype, device, args=args, architecture=arch.name, packed_weights=packed_weights,
                   memory_budget=memory_budget)

    @classmethod
    def from_folder(cls, model_dir: str | Path, dtype: torch.dtype, device: torch.device | str,
                    packed_weights: Optional[bool] = None, memory_budget: Optional[int] = None) -> "Model":
        """The model that ``config.json`` names, with the folder's weights."""
        model = cls.from_config(read_config_json(model_dir), dtype, device, packed_weights, memory_budget)
        model.load(SafetensorsSource(model_dir))
        return model

    @classmethod
    def random(cls, config: Mapping[str, Any], seed: int, dtype: torch.dtype,
               device: torch.device | str, packed_weights: Optional[bool] = None,
               memory_budget: Optional[int] = None) -> "Model":
        """Seeded random weights drawn on the device, without a folder."""
        model = cls.from_config(config, dtype, device, packed_weights, memory_budget)
        model.load(RandomSource(model.parts.tensor_specs(), seed, dtype, device))
        return model

    def load(self, source: TensorSource) -> None:
        specs = self.parts.tensor_specs()
        check_against_specs(source, specs, self.parts.duplicates())
        pack = self.packed_weights
        if pack is None:
            matrix_bytes = sum(math.prod(s.shape) for s in specs if s.role == MATRIX) * 2
            pack = self.dtype == torch.bfloat16 and packing_fits(matrix_bytes, self.device, self.memory_budget)
        with packing(pack and self.dtype == torch.bfloat16):
            for part in self.parts.all_parts:
                tensors = {s.name: source.get(s.name) for s in part.tensor_specs()}
                part.load(tensors, self.dtype, self.device)
            if getattr(self.parts.head, "tied_to", None):
                self.parts.head.tie(self.parts.embed.weight)
        self.loaded = True

    # ------------------------------------------------------------- needs
    def paged_needs(self) -> List[Optional[PagedNeed]]:
        """Per run entry: the pages it owns (None if it owns none)."""
        out: List[Optional[PagedNeed]] = []
        for e in self.layout.order:
            out.append(None if e.reads_cache_of is not None else self.parts.mixers[e.layer].paged_need())
        return out

    def state_needs(self) -> Dict[int, StateNeed]:
        out: Dict[int, StateNeed] = {}
        for i, e in enumerate(self.layout.order):
            need = None if e.reads_cache_of is not None else self.parts.mixers[e.layer].state_need()
            if need is not None:
                out[i] = need
        return out

    def capturable(self) -> bool:
        """Whether every part's forward may be recorded into a HIP graph."""
        return all(getattr(p, "capturable", True) for p in self.parts.all_parts)

    def packed(self) -> bool:
        """Whether the matrices have their second copy in the streaming kernels' order."""
        return any(isinstance(v, StreamedMatrix) and v.packed is not None
                   for p in self.parts.all_parts for v in vars(p).values())

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for p in self.parts.all_parts:
            for v in vars(p).values():
                held = [v.rows, v.packed.data if v.packed is not None else None] if isinstance(v, StreamedMatrix) else [v]
                for t in held:
                    if isinstance(t, torch.Tensor) and t.data_ptr() not in seen:
                        seen.add(t.data_ptr())
                        total += t.numel() * t.element_size()
        return total

    # ------------------------------------------------------------- forward
    def forward(self, ctx: StepContext, stores: Sequence[LayerStore]) -> Optional[torch.Tensor]:
        """Run the step's tokens through every entry of the order; fp32
        logits ``[n_out, vocab]`` at ``ctx.out_rows`` (None when none is wanted;
        the cache is written all the same)."""
        if not self.loaded:
            raise RuntimeError("the model has no weights yet")
        h = self.parts.embed.forward(ctx.tokens, ctx)
        pending = None  # rows still to be added to h, or ScaledRows (added already, the next norm half done)
        blocks, order = self.parts.blocks, self.layout.order
        for i, entry in enumerate(order):
            block = blocks[entry.layer]
            if getattr(block, "folds_norms", False):
                # the norm that follows this block is the next block's first, if that block can take over
                after = blocks[order[i + 1].layer] if i + 1 < len(order) else None
                next_norm = after.mixer_norm if getattr(after, "folds_norms", False) else None
                pending = block.forward(h, pending, ctx, stores[i], next_norm=next_norm)
            else:
                pending = block.forward(h, None if isinstance(pending, ScaledRows) else pending, ctx, stores[i])
        if isinstance(pending, ScaledRows):
            pending = None  # h holds the sum already
        if ctx.n_out == 0:
            return None
        x = self.parts.final_norm.forward(h, pending, ctx.act_dtype, rows=ctx.out_rows)
        return self.parts.head.forward(x)
