"""Choice of the next token from fp32 logits.

The reference (``fastgen/generate.py:887-896``, ``utils/sampling.py:6-31``):
greedy is ``argmax``; otherwise ``softmax(logits / temperature)`` and either a
plain multinomial draw (``top_p >= 1``) or a draw from the nucleus.  One global
switch decides greedy or not, and one global generator feeds every request.
Here every request carries its own temperature (0 = greedy), nucleus and seed;
the uniform number for its ``k``-th generated token is a function of
``(seed, k)`` alone, so what a request samples does not depend on its
batch-mates or on how its prompt was cut.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import torch

from ..kernels import ops


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 1.0
    seed: Optional[int] = None  # None: derived from the engine's seed and the request's arrival number
    max_new_tokens: int = 16
    stop_ids: Tuple[int, ...] = ()
    logprobs: bool = False
    # whether a request that ends on a stop id keeps it as its last token (the reference's
    # generator keeps it, fastgen/generate.py:647-662; its chat tool drops it, tools/chat.py:205-206)
    keep_stop_token: bool = True
    # a request whose prompt and max_new_tokens exceed the whole cache is refused, unless it
    # agrees to end early (the reference clamps every request so, fastgen/generate.py:95-113)
    truncate: bool = False


class Sampler:
    """Batches the per-request parameters and calls the sampling kernel."""

    def __init__(self, device: torch.device | str) -> None:
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
               seeds: Sequence[int], counters: Sequence[int]) -> torch.Tensor:
        """int32 ``[n]`` on the device; row ``i`` is greedy if ``temperatures[i] == 0``."""
        return self.prepare(temperatures, top_ps, seeds, counters, 1)(logits, 0, None)

    def prepare(self, temperatures: Sequence[float], top_ps: Sequence[float], seeds: Sequence[int],
                counters: Sequence[int], n_steps: int):
        """A function ``(logits, step, out) -> tokens`` for ``n_steps`` steps of
        the same rows, the parameters copied to the device once; the row's
        counter at step ``s`` is ``counters[row] + s``."""
        if not any(t > 0 for t in temperatures):
            return lambda logits, step, out: ops.sample(logits, out=out)
        packed_f = ops.upload([list(temperatures), list(top_ps)], torch.float32, self.device)
        mask = (1 << 63) - 1
        ints = [[s & mask for s in seeds]] + [[c + s for c in counters] for s in range(n_steps)]
        packed_i = ops.upload(ints, torch.int64, self.device)
        top_p = packed_f[1] if any(p < 1.0 for p in top_ps) else None
        return lambda logits, step, out: ops.sample(logits, packed_f[0], top_p, packed_i[0], packed_i[1 + step],
                                                    out=out)

    def logprobs(self, logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
        return ops.logprob(logits, tokens)
