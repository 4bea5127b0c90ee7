"""Shared by the GPU tests: model folders from plain weights, trace running,
and the tolerance rule."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, List, Mapping, Optional

import torch

from plain_llama import plain_forward


def save_model_folder(path: Path, config: Mapping, weights: Mapping[str, torch.Tensor],
                      dtype: torch.dtype = torch.float32) -> Path:
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    with open(path / "config.json", "w") as f:
        json.dump(dict(config), f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, str(path / "model.safetensors"))
    return path


def make_runner(folder: Path, dtype: torch.dtype, page_size: int, max_tokens: int, max_requests: int = 4):
    from fastgen_amd.engine import Model, ModelRunner

    model = Model.from_folder(folder, dtype, "cuda:0")
    return ModelRunner(model, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests)


def run_trace(runner, trace, tokens: Mapping[str, List[int]]) -> Dict[str, torch.Tensor]:
    """Logits of every fed token, per request ``[len, vocab]`` (fp32, CPU)."""
    from fastgen_amd.engine import StepEntry

    rows: Dict[str, List[torch.Tensor]] = {rid: [] for rid in tokens}
    for entries, ends in trace:
        step = [StepEntry(rid, tokens[rid][s : s + n], list(range(n))) for rid, s, n in entries]
        logits = runner.step(step).cpu()
        at = 0
        for rid, s, n in entries:
            assert len(rows[rid]) == s, f"{rid}: trace feeds position {s} after {len(rows[rid])}"
            rows[rid].extend(logits[at : at + n])
            at += n
        for rid in ends:
            runner.release(rid)
        runner.cache.check()
    return {rid: torch.stack(r) for rid, r in rows.items() if r}


def plain_logits(weights, config, tokens: Mapping[str, List[int]], dtype=torch.float32) -> Dict[str, torch.Tensor]:
    return {rid: plain_forward(weights, config, t, dtype) for rid, t in tokens.items()}


# the largest share of its tolerance that any comparison of this session has used, per precision
# (printed when the session ends: a creeping error shows here before it fails a test)
worst_share: Dict[str, tuple] = {}

# bfloat16: the share of the tolerance below that the engine may use.  The tolerance is twice the plain
# bfloat16 run's worst error over the request; the most that the engine has been seen to use of it, over all
# configurations and cuts, is 0.73 (portions of changing size at the smallest configuration), and what a
# session used at most is printed at its end.
BF16_SHARE = 0.9


def assert_close(got: Mapping[str, torch.Tensor], want: Mapping[str, torch.Tensor], dtype: torch.dtype,
                 noise: Optional[Mapping[str, torch.Tensor]] = None, what: str = "") -> float:
    """Returns the largest share of the tolerance that a position used.  float32: the engine and the plain implementation differ by rounding of
    fp32 sums only: 2e-5 of the largest logit; or, when ``want`` is a float64
    run and ``noise`` the plain float32 run (layers wide enough for the
    rounding of long sums to show), three times what the plain float32 run is
    off.  bfloat16: ``noise`` is the plain implementation run in bfloat16; the
    engine may be off the fp32 result by twice what that run is off, and no
    more."""
    share = 0.0
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape, f"{what} {rid}: shape {tuple(g.shape)} vs {tuple(w.shape)}"
        assert torch.isfinite(g).all(), f"{what} {rid}: non-finite logits"
        scale = float(w.abs().max())
        err = (g.double() - w.double()).abs().amax(dim=-1)  # per position
        w = w.to(torch.float32) if w.dtype == torch.float64 and dtype != torch.float32 else w
        if dtype == torch.float32 and noise is not None:
            tol = 3.0 * float((noise[rid].double() - w.double()).abs().max()) + 1e-6 * scale
        elif dtype == torch.float32:
            tol = 2e-5 * scale
        else:
            tol = 2.0 * float((noise[rid] - w).abs().max()) + 1e-3 * scale
            tol *= BF16_SHARE
        worst = int(err.argmax())
        assert float(err.max()) <= tol, (
            f"{what} request {rid}: first position over tolerance is "
            f"{int((err > tol).nonzero()[0])} of {len(err)}, worst {worst}: {float(err.max()):.3e} > {tol:.3e}"
            f" ({float(err.max()) / tol:.2f} of it)"
        )
        share = max(share, float(err.max()) / tol)
    key = str(dtype).replace("torch.", "")
    if share > worst_share.get(key, (0.0, ""))[0]:
        worst_share[key] = (share, what)
    return share


def write_tiny_tokenizer(folder: Path, n_words: int = 40) -> List[str]:
    """A word-level tokenizer (``tokenizer.json``, ``tokenizer_config.json`` with
    an end token and a chat template) in ``folder``; returns its words."""
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit

    words = ["<unk>", "<end>", "<user>", "<bot>"] + [f"w{i}" for i in range(n_words)]
    tok = Tokenizer(WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = WhitespaceSplit()
    tok.save(str(folder / "tokenizer.json"))
    template = "{% for m in messages %}{{ '<user> ' if m['role'] == 'user' else '<bot> ' }}{{ m['content'] }} <end> {% endfor %}<bot>"
    with open(folder / "tokenizer_config.json", "w") as f:
        json.dump({"eos_token": {"content": "<end>"}, "chat_template": template}, f)
    return words

