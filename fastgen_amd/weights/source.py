"""Where tensors come from: safetensors files of a model folder, a dict, or a
seeded random generator.  All three answer the same three questions (which
names, what shape, give me one), so the model loads from any of them.

The reference reads ``model-*-of-*.safetensors`` shard by shard and looks each
key up by name (``fastgen/utils/loading.py:255-293``); a single
``model.safetensors`` and an index file are accepted here as well.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Iterable, List, Mapping, Sequence, Tuple

import torch

from ..parts.base import TensorSpec


class WeightError(RuntimeError):
    """Checkpoint and model disagree; the message lists every disagreement."""


class TensorSource:
    def names(self) -> List[str]:
        raise NotImplementedError

    def shape(self, name: str) -> Tuple[int, ...]:
        raise NotImplementedError

    def get(self, name: str) -> torch.Tensor:
        raise NotImplementedError


class DictSource(TensorSource):
    def __init__(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self._t = dict(tensors)

    def names(self) -> List[str]:
        return list(self._t)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._t[name].shape)

    def get(self, name: str) -> torch.Tensor:
        return self._t[name]


def safetensors_files(model_dir: str | Path) -> List[Path]:
    d = Path(model_dir)
    index = d / "model.safetensors.index.json"
    if index.is_file():
        with open(index) as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
        return [d / f for f in files]
    single = d / "model.safetensors"
    if single.is_file():
        return [single]
    shards = sorted(d.glob("model-*-of-*.safetensors"))
    if shards:
        return shards
    raise WeightError(f"{d}: no model.safetensors, model.safetensors.index.json or model-*-of-*.safetensors")


class SafetensorsSource(TensorSource):
    """Tensors of a model folder, read lazily by name."""

    def __init__(self, model_dir: str | Path) -> None:
        from safetensors import safe_open

        self._files = safetensors_files(model_dir)
        self._handles = []
        self._where: Dict[str, int] = {}
        for i, path in enumerate(self._files):
            if not path.is_file():
                raise WeightError(f"{path} is named by the index but does not exist")
            h = safe_open(str(path), framework="pt", device="cpu")
            self._handles.append(h)
            for k in h.keys():
                if k in self._where:
                    raise WeightError(f"tensor {k!r} is stored in two files of {model_dir}")
                self._where[k] = i

    def names(self) -> List[str]:
        return list(self._where)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._handles[self._where[name]].get_slice(name).get_shape())

    def get(self, name: str) -> torch.Tensor:
        return self._handles[self._where[name]].get_tensor(name)


class RandomSource(TensorSource):
    """Seeded random tensors for a list of specs.

    Each tensor has a generator of its own, keyed by (seed, name), so its
    values do not depend on which other tensors exist or on the order asked.
    Matrices and tables are N(0, std); norm weights are 1 + N(0, std).
    Values are drawn in fp32 and then cast to ``dtype``.
    """

    def __init__(self, specs: Sequence[TensorSpec], seed: int, dtype: torch.dtype = torch.float32,
                 device: str | torch.device = "cpu") -> None:
        self._specs = {s.name: s for s in specs}
        self.seed, self.dtype, self.device = int(seed), dtype, torch.device(device)

    def names(self) -> List[str]:
        return list(self._specs)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._specs[name].shape)

    def get(self, name: str) -> torch.Tensor:
        spec = self._specs[name]
        key = hashlib.sha256(f"{self.seed}:{name}".encode()).digest()
        g = torch.Generator(device=self.device)
        g.manual_seed(int.from_bytes(key[:8], "little") & ((1 << 63) - 1))
        kind, std = spec.init
        t = torch.empty(spec.shape, dtype=torch.float32, device=self.device)
        t.normal_(0.0, std, generator=g)
        if kind == "one_plus_normal":
            t += 1.0
        elif kind != "normal":
            raise ValueError(f"unknown init {kind!r} for {name}")
        return t.to(self.dtype)


def check_against_specs(source: TensorSource, specs: Iterable[TensorSpec],
                        duplicates: Mapping[str, str] = {}) -> None:
    """One error for everything that is wrong: tensors the model needs and the
    checkpoint lacks, tensors the checkpoint has and the model does not know,
    and tensors of another shape than the configuration asks for.

    ``duplicates`` maps a name the checkpoint may carry to the tensor it must
    repeat (a tied head stored beside the embedding); such a tensor is
    tolerated only when both are equal.
    """
    want = {s.name: tuple(s.shape) for s in specs}
    have = set(source.names())
    missing = sorted(n for n in want if n not in have)
    unexpected = []
    for n in sorted(have - set(want)):
        twin = duplicates.get(n)
        if twin is not None and twin in have and source.shape(n) == source.shape(twin) \
                and torch.equal(source.get(n), source.get(twin)):
            continue
        unexpected.append(n)
    wrong = [(n, source.shape(n), want[n]) for n in sorted(want) if n in have and source.shape(n) != want[n]]
    if not (missing or unexpected or wrong):
        return
    lines = ["checkpoint does not fit the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}): " + ", ".join(
            f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in wrong))
    raise WeightError("\n".join(lines))
