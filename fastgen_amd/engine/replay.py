"""Trace replay: given token ids are fed through the model step by step and
the logits at the wanted places are written to disk.  Nothing is sampled.

It drives the same model, step function, cache and kernels that generation
uses (``ModelRunner.step``); it has no forward pass, cache or loader of its
own.  The reference has no such tool.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import IO, Optional

import torch

from ..config import read_config_json
from .context import StepEntry
from .model import Model
from .runner import ModelRunner

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, page_size: int = 64,
           stdin: Optional[IO[str]] = None, stdout: Optional[IO[str]] = None, max_live: int = 4,
           random_weights: Optional[int] = None) -> int:
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    if not torch.cuda.is_available():
        raise RuntimeError("trace_run needs a GPU: fastgen_amd has no CPU execution path")
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    if random_weights is None:
        model = Model.from_folder(model_dir, DTYPES[dtype], "cuda:0")
    else:  # the folder's (or the file's) configuration, tensors drawn on the device from the seed
        path = Path(model_dir)
        if path.is_file():
            with open(path) as f:
                config = json.load(f)
        else:
            config = read_config_json(path)
        model = Model.random(config, random_weights, DTYPES[dtype], "cuda:0")
    # each request's count is rounded up to whole pages of at least 64 tokens
    unit = max(64, page_size)
    pool_tokens = -(-max_tokens // unit) * unit
    runner = ModelRunner(model, page_size=page_size, max_tokens=pool_tokens, max_requests=max_live)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [
            StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
            for e in rec.get("entries", [])
        ]
        fresh = sum(1 for e in entries if not runner.cache.is_live(e.rid))
        if fresh > runner.cache.free_slots():
            raise RuntimeError(
                f"step {step}: {len(runner.cache.live_requests()) + fresh} requests would be live, --max-live is"
                f" {max_live}"
            )
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
                arr.tofile(out / f"{step}.f32")
        for rid in rec.get("end", []):
            if runner.cache.is_live(rid):
                runner.release(rid)
        torch.cuda.synchronize()
        print(f"done {step}", file=stdout, flush=True)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(
        prog="trace_run",
        description="Feed given token ids through a model step by step and write the logits asked for.",
    )
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=sorted(DTYPES))
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=64, help="tokens per cache page (default 64)")
    ap.add_argument("--max-live", type=int, default=4, help="most requests that are live at a time (default 4)")
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="read no weights: --model names a folder with config.json (or the file itself), the"
                         " tensors are drawn on the GPU from this seed")
    a = ap.parse_args(argv)
    if a.max_live < 1:
        ap.error("--max-live must be at least 1")
    return replay(a.model, a.dtype, a.out, a.max_tokens, a.page_size, max_live=a.max_live,
                  random_weights=a.random_weights)
