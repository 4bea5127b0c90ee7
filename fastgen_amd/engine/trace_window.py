"""A profiler trace of a few iterations of a running loop, on request.

The reference lets an operator ask a serving process for a trace without
stopping it (``fastgen/generate.py:187-196, 364-403``: a signal or a call,
``torch.profiler`` over the next iterations of the generation loop, a chrome
trace in a temporary folder).  Here that is one object which the loop ticks:
``request()`` may come from any thread or from a signal handler, ``tick()``
at the top of an iteration opens the profiler when a request is waiting and
closes it, writing the trace, once the window's iterations have passed.
"""

from __future__ import annotations

import contextlib
import logging
import os
import time
from typing import Any, Optional

logger = logging.getLogger("fastgen_amd")


class TraceWindow:
    def __init__(self, n_iters: int, out_dir: str, prefix: str = "fastgen") -> None:
        self.n_iters = max(1, int(n_iters))
        self.out_dir, self.prefix = out_dir, prefix
        self.last_path: Optional[str] = None  # the trace written last
        self._wanted = False  # a request that no tick has taken up yet (a plain store: safe in a signal handler)
        self._left = 0  # iterations the open window still covers
        self._stack: Optional[contextlib.ExitStack] = None
        self._profiler: Any = None

    @classmethod
    def from_env(cls) -> "TraceWindow":
        """FG_PROFILE_ITERS iterations (default 8) into FG_PROFILE_DIR (default /tmp), as the reference names them."""
        return cls(int(os.environ.get("FG_PROFILE_ITERS", "8")), os.environ.get("FG_PROFILE_DIR", "/tmp"))

    @property
    def pending(self) -> bool:
        return self._wanted

    @property
    def recording(self) -> bool:
        return self._stack is not None

    def request(self) -> None:
        """Ask for a trace of the next ``n_iters`` iterations; ignored while one is waiting or running."""
        if not self._wanted and not self.recording:
            self._wanted = True

    def tick(self) -> None:
        """Top of a loop iteration."""
        if self.recording:
            self._left -= 1
            if self._left <= 0:
                self.close()
        elif self._wanted:
            self._wanted = False
            self._open()

    def _open(self) -> None:
        from torch.profiler import ProfilerActivity, profile

        logger.info("tracing the next %d iterations", self.n_iters)
        stack = contextlib.ExitStack()
        self._profiler = stack.enter_context(
            profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA], with_stack=True))
        self._stack, self._left = stack, self.n_iters

    def close(self, write: bool = True) -> None:
        """End an open window (a loop that ends early calls this: the trace holds what there was)."""
        if not self.recording:
            return
        stack, prof = self._stack, self._profiler
        self._stack = self._profiler = None
        self._left = 0
        try:
            stack.close()
            if write:
                stamp = time.strftime("%H%M%S") + f".{int(time.time() * 1e6) % 1_000_000:06d}"
                path = os.path.join(self.out_dir, f"{self.prefix}_{os.getpid()}_{stamp}.json.gz")
                prof.export_chrome_trace(path)
                self.last_path = path
                logger.info("trace written to %s", path)
        except Exception as e:  # a trace that cannot be written must not end the loop it watched
            logger.warning("the trace could not be written: %r", e)
