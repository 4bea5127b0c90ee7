"""The reference's programming interface on top of the engine:
``GenArgs``, ``Packet`` and ``Fastgen.build(...).generate(queue)``
(``fastgen/generate.py:30-76, 138-173, 405-475``), with the same names and
meanings of options where the reference has them.

    fg = Fastgen.build(HfLoader(model_dir), GenArgs(max_batch=8, max_gen=64))     # or the folder itself
    q = queue.Queue(); q.put(Packet(thread_id=0, tokens=[1, 2, 3])); q.put(None)
    for pkt in fg.generate(q):
        print(pkt.thread_id, pkt.tokens)
"""

from __future__ import annotations

import logging
import os
import queue
import weakref
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Iterator, List, Optional, Sequence

import torch

from .engine import Engine, Model
from .engine.trace_window import TraceWindow
from .sampling import SamplingParams

logger = logging.getLogger(__name__)


@dataclass
class GenArgs:
    """Generation options (``fastgen/generate.py:30-59``).  Options of the
    reference that belong to parts this engine does not have (fp8 clipping,
    the hold-back thresholds ``min_prefill`` / ``min_prefill_batch``, which
    with the reference's defaults never hold anything back) are absent."""

    use_sampling: bool = True  # else greedy for every request
    temperature: float = 0.7
    top_p: float = 0.9
    logprobs: bool = False
    max_batch: int = 256  # most concurrent requests
    max_seq: int = -1  # cache size in tokens, also the cap of one request; negative: from gpu_gb
    max_gen: Optional[int] = None  # default cap of generated tokens
    host_cache_gb: float = 0  # the reference's host-memory prefix cache: not built, must stay 0
    cache_block: int = 64  # tokens per cache page (the reference's default is 256)
    num_cuda_graphs: int = 64  # most captured decode steps (the reference: 16); 0: every step runs eagerly
    max_prefill: int = 8192  # token budget of one step
    prefill_gb: float = 0.5  # activation budget, used when sizing the cache
    gpu_gb: float = 20  # memory budget, used when max_seq is negative; 0 or less: all that the GPU has free
    sync_freq: int = 10  # decode steps between host checks for finished requests (when nobody waits)
    seed: int = 777  # the reference's tools seed the global generator with 777 (tools/chat.py:47)
    dtype: torch.dtype = torch.bfloat16


@dataclass
class Packet:
    """A request going in, a generation coming out (``fastgen/generate.py:62-76``)."""

    thread_id: Any
    tokens: List[int] = field(default_factory=list)
    temperature: Optional[float] = None
    logprobs: Optional[List[float]] = None
    max_gen: Optional[int] = None
    error: Optional[str] = None  # set on a packet that comes back refused (not in the reference)


def cache_tokens_for_budget(model: Model, gen_args: GenArgs, bytes_per_token: int) -> int:
    """``fastgen/utils/tune.py:68-84``: what is left of ``gpu_gb`` after the
    weights and the activation budget, in tokens of cache, rounded up to a page."""
    left = gen_args.gpu_gb * 1e9 - model.weight_bytes() - gen_args.prefill_gb * 1e9
    tokens = int(left // max(1, bytes_per_token))
    if tokens < gen_args.cache_block:
        raise RuntimeError(
            f"gpu_gb={gen_args.gpu_gb} leaves no room for one cache page beside"
            f" {model.weight_bytes() / 1e9:.2f} GB of weights"
        )
    return -(-tokens // gen_args.cache_block) * gen_args.cache_block


def memory_budget(gen_args: GenArgs) -> Optional[int]:
    """The bytes that the weights and the cache share, where the arguments name them (``gpu_gb`` sizes the
    cache): a model loaded for these arguments makes its second copy of the matrices
    (``kernels.linear.StreamedMatrix``) only if that leaves half of the budget to the cache.  None: the
    GPU's memory is the budget."""
    return int(gen_args.gpu_gb * 1e9) if gen_args.max_seq < 0 and gen_args.gpu_gb > 0 else None


class HfLoader:
    """A model folder in the Hugging Face layout: ``config.json``,
    ``model.safetensors`` (or shards with an index) and, optionally,
    ``tokenizer.json`` (``fastgen/utils/loading.py:203-260``; only local
    folders: nothing is fetched)."""

    def __init__(self, model: str | Path) -> None:
        self.model_dir = Path(model)
        if not (self.model_dir / "config.json").is_file():
            raise FileNotFoundError(f"{self.model_dir}: no config.json (a model folder is needed; hub ids are not fetched)")

    def load_model_args(self):
        """The typed configuration of the folder's architecture."""
        import json

        from .config import get_architecture

        with open(self.model_dir / "config.json") as f:
            config = json.load(f)
        return get_architecture(config).parse(config)

    def load_tokenizer(self):
        """The folder's tokenizer, or None if it has none."""
        from .tools.tokenizer import FolderTokenizer

        return FolderTokenizer.maybe(self.model_dir)


# The engine that SIGUSR2 asks for a trace: the one built last, held weakly, so that an engine that its
# owner has dropped gives its memory back and a later one gets the signal.
_signalled: Optional["weakref.ref[Fastgen]"] = None


def _on_profile_signal(_signum, _frame) -> None:
    fg = _signalled() if _signalled is not None else None
    if fg is not None:
        fg.request_profile()


def _route_profile_signal_to(fg: "Fastgen", signum: Optional[int] = None) -> None:
    """SIGUSR2 requests a trace from ``fg``, if nobody else handles that signal
    (``fastgen/generate.py:165-172``) and this is the main thread (only there can a handler be set)."""
    import signal
    import threading

    global _signalled
    signum = signal.SIGUSR2 if signum is None else signum
    if threading.current_thread() is not threading.main_thread():
        return
    current = signal.getsignal(signum)
    if current is not signal.SIG_DFL and current is not _on_profile_signal:
        logger.warning("a handler for signal %s is set; the profile handler was not installed", signum)
        return
    _signalled = weakref.ref(fg)
    if current is signal.SIG_DFL:
        signal.signal(signum, _on_profile_signal)


class Fastgen:
    def __init__(self, engine: Engine, gen_args: GenArgs, stop_tokens: Sequence[int] = ()) -> None:
        self.engine, self.gen_args, self.stop_tokens = engine, gen_args, tuple(stop_tokens)
        # a trace on request: ``request_profile()``, or the signal SIGUSR2 where ``build`` could install
        # its handler (see ``engine.trace_window``)
        self.trace = TraceWindow.from_env()

    @classmethod
    def build(cls, loader: "HfLoader | str | Path", gen_args: GenArgs = GenArgs(), tp_mesh: Any = None,
              device: str = "cuda:0", stop_tokens: Optional[Sequence[int]] = None) -> "Fastgen":
        """Load the model of ``loader`` (an :class:`HfLoader` or the folder
        itself) and size its cache (``fastgen/generate.py:139-173``).
        ``tp_mesh`` is the reference's tensor-parallel mesh: this engine runs
        on one GPU and takes None only."""
        if tp_mesh is not None:
            raise RuntimeError("fastgen_amd runs on one GPU: tp_mesh must be None")
        model_dir = loader.model_dir if isinstance(loader, HfLoader) else loader
        device_ = torch.device(device)
        if device_.type != "cuda":
            raise RuntimeError("fastgen_amd runs on a GPU only")  # generate.py:148
        model = Model.from_folder(model_dir, gen_args.dtype, device_, memory_budget=memory_budget(gen_args))
        if stop_tokens is None and isinstance(loader, HfLoader):
            tokenizer = loader.load_tokenizer()
            stop_tokens = tokenizer.stop_tokens if tokenizer is not None else None
        return cls.from_model(model, gen_args, stop_tokens)

    @classmethod
    def from_model(cls, model: Model, gen_args: GenArgs = GenArgs(),
                   stop_tokens: Optional[Sequence[int]] = None, num_pages: Optional[int] = None) -> "Fastgen":
        """Size the cache for a model that is already on the device (``fastgen/generate.py:206-244``):
        ``num_pages`` pages if given, else ``max_seq`` tokens, else what ``gpu_gb`` leaves beside the
        weights, else (``gpu_gb <= 0``) what the device has free."""
        if gen_args.host_cache_gb:
            raise RuntimeError("fastgen_amd has no host-memory prefix cache: host_cache_gb must be 0")
        if stop_tokens is None:
            eos = getattr(model.args, "extra", {}).get("eos_token_id", [])
            stop_tokens = eos if isinstance(eos, (list, tuple)) else [eos]
        max_tokens: Optional[int] = gen_args.max_seq
        if num_pages is not None:
            if num_pages < 1:
                raise ValueError("num_pages must be at least 1")
            max_tokens = num_pages * gen_args.cache_block
        elif gen_args.max_seq < 0:
            if gen_args.gpu_gb > 0:
                esize = torch.empty((), dtype=gen_args.dtype).element_size()
                per_token = sum(n.n_kv_heads * (n.head_dim + n.value_dim) * esize
                                for n in model.paged_needs() if n is not None)
                max_tokens = cache_tokens_for_budget(model, gen_args, per_token)
            else:
                max_tokens = None  # the engine takes what is free
        max_batch = gen_args.max_batch
        if max_tokens is not None:
            max_batch = max(1, min(max_batch, max_tokens // gen_args.cache_block))  # generate.py:234-236
        engine = Engine(model, page_size=gen_args.cache_block, max_tokens=max_tokens, max_batch=max_batch,
                        max_step_tokens=gen_args.max_prefill, max_seq=max_tokens, seed=gen_args.seed,
                        sync_freq=gen_args.sync_freq, reserve_bytes=int(gen_args.prefill_gb * 1e9) + (2 << 30)
                        if max_tokens is None else None)
        logger.info("cache of %d tokens in pages of %d, at most %d requests",
                    engine.scheduler.pool_tokens, gen_args.cache_block, engine.scheduler.max_batch)
        engine.runner.max_graphs = max(0, gen_args.num_cuda_graphs)
        fg = cls(engine, gen_args, stop_tokens)
        _route_profile_signal_to(fg)
        return fg

    # ---------------------------------------------------------- profiling
    def request_profile(self) -> None:
        """Ask for a trace of the next ``FG_PROFILE_ITERS`` iterations of the generation loop (the
        reference's hook of the same name, ``fastgen/generate.py:187-196``)."""
        self.trace.request()

    def _params(self, pkt: Packet) -> SamplingParams:
        ga = self.gen_args
        # as in the reference a packet's temperature of None or 0 falls back to
        # the default (generate.py:790); greedy is the global switch (892)
        temp = (pkt.temperature or ga.temperature) if ga.use_sampling else 0.0
        max_gen = pkt.max_gen or ga.max_gen or (self.engine.scheduler.max_seq - len(pkt.tokens))
        # maxlen = min(len + max_gen, max_seq) (generate.py:95-113): a request is cut short, not refused
        return SamplingParams(temperature=temp, top_p=ga.top_p, max_new_tokens=max(1, max_gen),
                              stop_ids=self.stop_tokens, logprobs=ga.logprobs, truncate=True)

    def generate(self, q: "queue.Queue[Optional[Packet]]") -> Iterator[Packet]:
        """Packets from ``q`` in, finished packets out, in the order they
        finish; ``None`` on the queue ends the input, and what is in flight
        completes (``fastgen/generate.py:405-425``).  Blocks on the queue only
        when nothing is in flight (547)."""
        eoq = False
        pending = {}
        refused: List[Packet] = []
        while True:
            self.trace.tick()
            while not eoq:
                try:
                    pkt = q.get(block=not self.engine.has_work())
                except queue.Empty:
                    break
                if pkt is None:
                    eoq = True
                    break
                try:
                    rid = self.engine.add_request(pkt.tokens, self._params(pkt))
                except ValueError as e:
                    # one caller's bad packet (empty, too long, an id outside the vocabulary) does not
                    # end the others': it comes back at once, without tokens, the reason in ``error``
                    logger.warning("packet %r refused: %s", pkt.thread_id, e)
                    refused.append(Packet(thread_id=pkt.thread_id, tokens=[], temperature=pkt.temperature,
                                          logprobs=None, max_gen=pkt.max_gen, error=str(e)))
                    continue
                pending[rid] = pkt
            while refused:
                yield refused.pop(0)
            if not self.engine.has_work():
                if eoq:
                    self.trace.close()  # a trace that was still running is written with what it has
                    return
                continue
            for req in self.engine.step():
                src = pending.pop(req.rid)
                yield Packet(thread_id=src.thread_id, tokens=list(req.generated), temperature=src.temperature,
                             logprobs=list(req.logprobs) if self.gen_args.logprobs else None, max_gen=src.max_gen)

    def destroy(self) -> None:
        """Give the GPU memory back (``fastgen/generate.py:355-362``)."""
        self.engine = None  # type: ignore[assignment]
        torch.cuda.empty_cache()
