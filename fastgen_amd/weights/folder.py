"""Writing a model folder: ``config.json`` and ``model.safetensors`` from a
configuration and a seed (the random-weights mode).  The reference has no
such mode; it creates parameters on the meta device and fills them from a
checkpoint only (``fastgen/generate.py:155-160``)."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping, Optional

import torch

from ..config import get_architecture
from ..config.layout import ModelLayout
from .source import RandomSource


def layout_tensor_specs(layout: ModelLayout):
    """Tensor specs of a layout, without placing anything on a device."""
    from ..engine.model import build_parts

    return build_parts(layout).tensor_specs()


def write_model_folder(model_dir: str | Path, config: Mapping[str, Any] | Any, seed: int,
                       dtype: torch.dtype = torch.float32, architecture: Optional[str] = None) -> Path:
    """Write ``config.json`` and ``model.safetensors`` with seeded random
    weights under the checkpoint's tensor names.

    ``config`` is either the dict of ``config.json`` keys or the typed record
    of the architecture (then ``architecture`` names it).
    """
    from safetensors.torch import save_file

    if isinstance(config, Mapping):
        arch = get_architecture(architecture or config)
        args = arch.parse(config)
    else:
        arch = get_architecture(architecture or getattr(config, "architecture"))
        args = config
    out = Path(model_dir)
    out.mkdir(parents=True, exist_ok=True)
    hf = arch.to_hf_config(args)
    hf["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16"}[dtype]
    with open(out / "config.json", "w") as f:
        json.dump(hf, f, indent=2)
    specs = layout_tensor_specs(arch.layout(args))
    src = RandomSource(specs, seed, dtype)
    save_file({s.name: src.get(s.name).contiguous() for s in specs}, str(out / "model.safetensors"),
              metadata={"format": "pt"})
    return out
