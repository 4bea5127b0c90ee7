"""The engine: a model with its cache, the scheduler above the step function,
and sampling.  ``add_request`` / ``step`` for a serving loop, ``generate`` for
a batch of prompts.  (The reference's counterpart is ``Fastgen`` in
``fastgen/generate.py:138-475``; ``fastgen_amd.generate`` offers that
interface on top of this class.)
"""

from __future__ import annotations

import logging
import os
import time
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, Hashable, List, Mapping, Optional, Sequence

import torch

from ..sampling import Sampler, SamplingParams
from .context import StepEntry
from .model import Model
from .runner import ModelRunner
from .scheduler import PENDING, PlannedEntry, Request, Scheduler


logger = logging.getLogger("fastgen_amd")


@dataclass
class _InFlight:
    """A step whose samples the host has not seen yet."""

    plan: List[PlannedEntry]
    tokens: torch.Tensor  # int32 [rows] on the device: what the next step's entries take their tokens from
    row_of: Dict[int, int]  # id(request) -> its row
    host_tokens: torch.Tensor  # pinned copy, complete once ``copied`` has happened
    host_logprobs: Optional[torch.Tensor]
    copied: torch.cuda.Event


def step_memory_estimate(model: Model, max_step_tokens: int, max_batch: int) -> int:
    """Bytes that one step's intermediate tensors take at most: per token a few rows as wide as the
    widest matrix product of a layer (its output, the activation made from it, the fp32 partial sums
    of the product after it) and the fp32 residual stream; per request a row of fp32 logits, twice
    (a captured step keeps its own).  (``fastgen/utils/tune.py:46-65`` budgets 1.2 x (4 dim + 4 ffn)
    bytes a token for the same purpose.)"""
    widest = model.layout.dim
    for part in model.parts.all_parts[1:-1]:  # the layers' parts; the embedding and the head are not per token
        for v in vars(part).values():
            shape = getattr(v, "shape", None)  # a tensor or a kernels.linear.StreamedMatrix
            if shape is not None and len(shape) == 2:
                widest = max(widest, shape[0])
    return int(max_step_tokens * 12 * widest + 3 * max_batch * model.vocab_size * 4)


@dataclass
class WorkDone:
    """What the engine's steps have asked of the GPU so far, for measurements: ``steps`` runs of the model
    (each reads every weight once), ``tokens`` run through it, ``cache_reads``: over all steps and their
    requests, the cached tokens of the request after the step (what its attention reads at least once),
    ``keys_attended``: over all tokens, the keys each attends (its attention's products)."""

    steps: int = 0
    tokens: int = 0
    cache_reads: int = 0
    keys_attended: int = 0

    def note(self, start: int, n: int) -> None:
        """A request brought ``n`` tokens at positions ``start ..`` to one step."""
        self.tokens += n
        self.cache_reads += start + n
        self.keys_attended += n * start + n * (n + 1) // 2


class Engine:
    def __init__(self, model: Model, page_size: int = 64, max_tokens: Optional[int] = 8192, max_batch: int = 64,
                 max_step_tokens: int = 2048, max_seq: Optional[int] = None, seed: int = 0,
                 sync_freq: int = 10, overlap_steps: Optional[bool] = None,
                 reserve_bytes: Optional[int] = None, admit_reserve: int = 128) -> None:
        """``max_tokens``: the cache's size in tokens; None: whatever memory the device has free
        now, the weights being in place, beside ``reserve_bytes`` (default: an estimate of what a
        step of ``max_step_tokens`` tokens and ``max_batch`` rows of logits take, plus 2 GiB).
        ``admit_reserve``: tokens of growth that admission keeps room for (see ``Scheduler``)."""
        self.model = model
        cap = getattr(model.args, "max_position", 0) or None
        if max_seq is None:
            max_seq = cap
        elif cap:
            max_seq = min(max_seq, cap)
        if reserve_bytes is None:
            reserve_bytes = step_memory_estimate(model, max_step_tokens, max_batch) + (2 << 30)
        at_most = max_batch * (-(-max_seq // page_size) * page_size) if max_seq else None
        self.runner = ModelRunner(model, page_size=page_size, max_tokens=max_tokens, max_requests=max_batch,
                                  reserve_bytes=reserve_bytes, at_most_tokens=at_most)
        self.scheduler = Scheduler(self.runner.cache, max_batch, max_step_tokens, max_seq, on_admit=self.runner.admit,
                                   admit_reserve=admit_reserve)
        # no request gets longer than the scheduler lets it: block tables need not be wider
        self.runner.table_width = min(self.runner.table_width, -(-self.scheduler.max_seq // page_size))
        self.sampler = Sampler(model.device)
        self.seed = seed
        # decode steps between host checks for finished requests when nothing waits for admission
        # (the reference's GenArgs.sync_freq, fastgen/generate.py:55-59)
        self.sync_freq = sync_freq
        # The host runs one step behind the device: a step is planned and launched from the counts of
        # tokens alone, the step before it hands its samples over on the device, and the host looks
        # at them (stop ids, the caller's lists) while the new step runs.  FG_NO_OVERLAP=1 (or False
        # here) makes every step wait for its tokens.
        if overlap_steps is None:
            overlap_steps = os.environ.get("FG_NO_OVERLAP", "0") in ("", "0")
        self.overlap_steps = overlap_steps
        self._in_flight: Optional[_InFlight] = None
        self._held: List[Request] = []  # ended, with samples still on the device
        self._n_requests = 0
        self._logged_running = -1  # the batch size that the log line of the last decode run named
        self.work = WorkDone()
        self.n_steps = 0
        self.last_mean_context = 0.0  # set by time_decode

    # -------------------------------------------------------------- build
    @classmethod
    def from_folder(cls, model_dir: str | Path, dtype: torch.dtype = torch.bfloat16, device: str = "cuda:0",
                    **kw: Any) -> "Engine":
        return cls(Model.from_folder(model_dir, dtype, device), **kw)

    @classmethod
    def from_config(cls, config: Mapping[str, Any], seed: int, dtype: torch.dtype = torch.bfloat16,
                    device: str = "cuda:0", **kw: Any) -> "Engine":
        """A model of this configuration with seeded random weights."""
        return cls(Model.random(config, seed, dtype, device), **kw)

    # ------------------------------------------------------------ serving
    def add_request(self, prompt: Sequence[int], params: SamplingParams = SamplingParams(),
                    rid: Optional[Hashable] = None) -> Hashable:
        rid = self._n_requests if rid is None else rid
        vocab = self.model.vocab_size
        if any(not 0 <= int(t) < vocab for t in prompt):
            raise ValueError(f"request {rid!r}: token id outside [0, {vocab})")
        # a request's own seed, unless it gave one: the engine's seed and its arrival number
        seed = params.seed if params.seed is not None else (self.seed * 1000003 + self._n_requests + 1)
        self._n_requests += 1
        self.scheduler.add(Request(
            rid=rid, prompt=[int(t) for t in prompt], max_new=params.max_new_tokens,
            temperature=float(params.temperature), top_p=float(params.top_p), seed=seed,
            stop_ids=tuple(params.stop_ids), want_logprobs=params.logprobs, truncate=params.truncate,
            keep_stop_token=params.keep_stop_token,
        ))
        return rid

    def has_work(self) -> bool:
        return self.scheduler.has_work() or self._in_flight is not None or bool(self._held)

    def abort(self, rid: Hashable) -> bool:
        """End a request before it is done; it comes out of the next ``step`` with ``finish_reason``
        ``aborted`` and what it has generated so far."""
        return self.scheduler.abort(rid)

    def step(self) -> List[Request]:
        """One step of the model over what the scheduler picks; the requests
        that ended and whose tokens the host has all seen (with overlapped steps
        a request is reported a step after its last one)."""
        sched = self.scheduler
        if self.runner.can_graph(len(sched.running)):
            if self._in_flight is not None and self._decode_run_ahead():
                self._settle()  # a decode run starts from tokens the host knows; a stop id among them may end one
            n_run = sched.plan_decode_run(self.sync_freq)
            if n_run:
                if len(sched.running) != self._logged_running:  # (the reference logs its active lanes so)
                    self._logged_running = len(sched.running)
                    logger.info("%d running, decoding %d steps at a time", self._logged_running, n_run)
                return self._ended(self._decode_run(n_run))
        plan = sched.plan()
        if not plan:
            self._settle()
            return self._ended([])
        entries, rows = [], []
        prev = self._in_flight
        for e in plan:
            toks = e.request.tokens_from(e.start, e.n)
            from_row = None
            if PENDING in toks:
                if e.n != 1 or prev is None:  # only ever the one token of a decoding request
                    raise RuntimeError(f"request {e.request.rid!r}: a portion holds a token the host has not seen")
                from_row, toks = prev.row_of[id(e.request)], [0]
            entries.append(StepEntry(e.request.rid, toks, [e.n - 1] if e.wants_logits else [], from_row))
            if e.wants_logits:
                rows.append(e.request)
        if logger.isEnabledFor(logging.INFO):
            self._logged_running = -1
            n_tokens = sum(e.n for e in plan)
            logger.info("step %d: %d running, %d waiting, %d tokens (%d of prompts)", self.n_steps,
                        len(sched.running), len(sched.waiting), n_tokens, n_tokens - len(rows))
        logits = self.runner.step(entries, prev.tokens if prev is not None else None)
        self.n_steps += 1
        self.work.steps += 1
        for e in plan:
            self.work.note(e.start, e.n)
        tok = lps = None
        if rows:
            tok = self.sampler.sample(
                logits, [r.temperature for r in rows], [r.top_p for r in rows], [r.seed for r in rows],
                [len(r.generated) for r in rows],
            )
            if any(r.want_logprobs for r in rows):
                lps = self.sampler.logprobs(logits, tok)
        if not rows:  # portions of prompts only: nothing to wait for
            done = sched.commit(plan, [])
            self._settle()
            return self._ended(done)
        if not self.overlap_steps:
            done = sched.commit(plan, tok.tolist(), lps.tolist() if lps is not None else None)
            return self._ended(done)
        host_tok = torch.empty(tok.shape, dtype=tok.dtype, pin_memory=True)
        host_tok.copy_(tok, non_blocking=True)
        host_lps = None
        if lps is not None:
            host_lps = torch.empty(lps.shape, dtype=lps.dtype, pin_memory=True)
            host_lps.copy_(lps, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        done = sched.commit(plan)  # its samples stay on the device for now
        self._in_flight = _InFlight(plan, tok, {id(r): i for i, r in enumerate(rows)}, host_tok, host_lps, copied)
        if prev is not None:
            self._resolve(prev)  # the step before: its tokens have long arrived
        return self._ended(done)

    def _decode_run_ahead(self) -> bool:
        """Whether a decode run would start once the step in flight is settled."""
        sched = self.scheduler
        return bool(sched.running) and not sched.waiting and all(r.remaining() == 1 for r in sched.running)

    def _resolve(self, step: _InFlight) -> None:
        step.copied.synchronize()
        self.scheduler.resolve(step.plan, step.host_tokens.tolist(),
                               step.host_logprobs.tolist() if step.host_logprobs is not None else None)

    def _settle(self) -> None:
        """Wait for the samples of the step in flight and let the scheduler see them."""
        if self._in_flight is not None:
            step, self._in_flight = self._in_flight, None
            self._resolve(step)

    def _ended(self, done: List[Request]) -> List[Request]:
        """``done`` and what else the scheduler ended since the last step (a request alone and out
        of pages ends while planning, a stop id ends one a step late); every ended request is
        reported once, when the host has seen all its tokens."""
        for r in done + self.scheduler.finished:
            if not any(r is h for h in self._held):
                self._held.append(r)
        self.scheduler.finished.clear()
        out = [r for r in self._held if r.n_pending == 0]
        self._held = [r for r in self._held if r.n_pending]
        for r in out:
            if (r.finish_reason == "stop" and not r.keep_stop_token and r.generated
                    and r.generated[-1] in r.stop_ids):
                r.generated.pop()
                del r.logprobs[len(r.generated):]
        return out

    def _decode_run(self, n_steps: int) -> List[Request]:
        """``n_steps`` decode steps of all running requests with one look at the
        tokens at the end."""
        reqs = list(self.scheduler.running)
        self.work.steps += n_steps
        for r in reqs:
            at = self.runner.cache.length(r.rid)  # the position of the token it brings to the first step
            for s_ in range(n_steps):
                self.work.note(at + s_, 1)
        entries = [StepEntry(r.rid, [r.generated[-1] if r.generated else r.prompt[-1]], [0]) for r in reqs]
        sample = self.sampler.prepare([r.temperature for r in reqs], [r.top_p for r in reqs],
                                      [r.seed for r in reqs], [len(r.generated) for r in reqs], n_steps)
        want_lp = any(r.want_logprobs for r in reqs)
        lps: List[torch.Tensor] = []

        def sample_and_note(logits, step, out):
            tok = sample(logits, step, out)
            if want_lp:
                lps.append(self.sampler.logprobs(logits, tok))
            return tok

        out = self.runner.decode_run(entries, n_steps, sample_and_note)
        tokens = out.tolist()  # the one synchronisation of the run
        self.n_steps += len(tokens)
        return self.scheduler.commit_run(tokens, [lp.tolist() for lp in lps] if want_lp else None)

    def generate(self, prompts: Sequence[Sequence[int]], params: SamplingParams | Sequence[SamplingParams] = SamplingParams(),
                 ) -> List[List[int]]:
        """Generated ids for every prompt, in the order of the prompts."""
        plist = list(params) if isinstance(params, (list, tuple)) else [params] * len(prompts)
        rids: List[Hashable] = []
        try:
            for p, sp in zip(prompts, plist):
                rids.append(self.add_request(p, sp))
        except Exception:
            for rid in rids:  # all or nothing: a refused prompt leaves none of the call's requests behind
                self.abort(rid)
            self.scheduler.finished.clear()
            raise
        out: Dict[Hashable, List[int]] = {}
        while self.has_work():
            for r in self.step():
                out[r.rid] = r.generated
        return [out[r] for r in rids]

    # ------------------------------------------------------- measurement
    def time_prefill(self, prompt: Sequence[int], repeats: int = 3) -> List[float]:
        """Seconds of one step that takes the whole prompt and returns the
        logits of its last token: each of ``repeats`` runs after one warm-up."""
        times: List[float] = []
        for i in range(repeats + 1):
            rid = ("prefill-timing", i)
            entry = StepEntry(rid, list(prompt), [len(prompt) - 1])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            self.runner.step([entry])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            self.runner.release(rid)
            if i:
                times.append(dt)
        return times

    def time_decode(self, prompts: Sequence[Sequence[int]], steps: int, warmup: int) -> float:
        """Seconds of exactly ``steps`` decode steps of the batch ``prompts``
        (greedy, no stop ids), after the prompts are in the cache and after
        ``warmup`` untimed decode steps."""
        # the first requests decode while the later prompts are still being fed: none may end
        # before the timed steps are over
        n_prompt_tokens = sum(len(p) for p in prompts)
        feed_steps = -(-n_prompt_tokens // max(1, self.scheduler.max_step_tokens - len(prompts))) + len(prompts)
        params = SamplingParams(temperature=0.0, max_new_tokens=feed_steps + warmup + steps + 8)
        for p in prompts:
            self.add_request(p, params)
        while any(r.remaining() > 1 for r in self.scheduler.running) or self.scheduler.waiting:
            self.step()
        def run(n: int) -> None:  # exactly n decode steps, in runs of sync_freq where the engine takes them
            target = self.n_steps + n
            keep = self.sync_freq
            while self.n_steps < target:
                self.sync_freq = min(keep, target - self.n_steps)
                if self.step():
                    raise RuntimeError("time_decode: a request ended inside the measurement")
            self.sync_freq = keep

        run(warmup)
        if len(self.scheduler.running) != len(prompts) or self.scheduler.n_preemptions:
            raise RuntimeError("time_decode: the batch did not stay whole; give the cache more pages")
        cached = lambda: sum(self.runner.cache.length(r.rid) for r in self.scheduler.running) / len(prompts)
        before = cached()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # tokens a request had in the cache, on average over the requests and the timed steps (the first
        # requests decoded while the later prompts were fed, so they are longer than their prompts)
        self.last_mean_context = (before + cached()) / 2
        for r in list(self.scheduler.running):  # the measurement is over: let go of the batch
            self.abort(r.rid)
        self._settle()
        self.scheduler.finished.clear()
        self._held.clear()
        return dt
