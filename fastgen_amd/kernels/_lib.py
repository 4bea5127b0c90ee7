"""Builds and loads the HIP kernel libraries.

Each file under ``fastgen_amd/csrc`` becomes one shared library with a plain
C interface, compiled by ``hipcc`` for gfx950 and loaded with ``ctypes``.  A
library is compiled the first time one of its kernels is asked for and kept
beside the package (or under the temporary directory when the package is not
writable); its file name carries a hash of the sources and flags, so a changed
source is rebuilt and a built one is found again.  There is no fallback: if a
library can be neither found nor built, the call raises.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import threading
import time
from pathlib import Path
from typing import Dict, Iterable, Optional

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HEADERS = ["common.h", "kv_layout.h", "attention_static.h"]

# library name -> source file
LIBRARIES: Dict[str, str] = {
    "rows": "rows.hip",
    "rope_kv": "rope_kv.hip",
    "attention": "attention.hip",
    "gemm": "gemm.hip",
    "gemm_skinny": "gemm_skinny.hip",
    "gemm_tiled": "gemm_tiled.hip",
    "sampling": "sampling.hip",
}

# libraries compiled once per value of a macro: name -> (source, macro, values that build_all compiles)
VARIANT_LIBRARIES: Dict[str, tuple] = {
    "attention_mfma": ("attention_mfma.hip", "FG_HD", tuple(range(16, 257, 16))),
}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (
        os.environ.get("HIPCC"),
        shutil.which("hipcc"),
        os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc"),
    ):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError(
        "hipcc was not found (looked at $HIPCC, PATH and $ROCM_PATH/bin): the HIP kernels"
        " of fastgen_amd cannot be built, and there is no other execution path"
    )


def _split_variant(name: str):
    """``attention_mfma@128`` -> (source file, ["-DFG_HD=128"], file stem)."""
    if "@" in name:
        base, value = name.split("@", 1)
        src, macro, _ = VARIANT_LIBRARIES[base]
        return src, [f"-D{macro}={int(value)}"], f"{base}_{int(value)}"
    return LIBRARIES[name], [], name


def _source_hash(name: str) -> str:
    src, defines, _ = _split_variant(name)
    h = hashlib.sha256()
    for f in [src, *HEADERS]:
        h.update(f.encode())
        h.update((CSRC / f).read_bytes())
    h.update(" ".join(HIPCC_FLAGS + defines).encode())
    return h.hexdigest()[:12]


def _build_dirs() -> Iterable[Path]:
    yield Path(__file__).resolve().parent.parent / "_built"
    tmp = os.environ.get("TMPDIR") or "/tmp"
    yield Path(tmp) / f"fastgen_amd-{os.getuid()}" / "_built"


def _lib_filename(name: str) -> str:
    return f"libfg_{_split_variant(name)[2]}-{_source_hash(name)}.so"


def find_built(name: str) -> Optional[Path]:
    fn = _lib_filename(name)
    for d in _build_dirs():
        if (d / fn).is_file():
            return d / fn
    return None


def _writable_dir() -> Path:
    last: Optional[Exception] = None
    for d in _build_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe-{os.getpid()}-{threading.get_ident()}"
            probe.write_bytes(b"")
            probe.unlink()
            return d
        except OSError as e:
            last = e
    raise KernelBuildError(f"no writable directory for built kernels: {last}")


def compile_library(name: str, *, verbose: bool = True) -> Path:
    """Compile one library now (also when a built one exists) and return its path."""
    src_name, defines, stem = _split_variant(name)
    src = CSRC / src_name
    out_dir = _writable_dir()
    out = out_dir / _lib_filename(name)
    tmp_out = out_dir / f".{out.name}.{os.getpid()}-{threading.get_ident()}.tmp"
    cmd = [_hipcc(), *HIPCC_FLAGS, *defines, f"-I{CSRC}", str(src), "-o", str(tmp_out)]
    if verbose:
        print(f"[fastgen_amd] compiling {src.name} {' '.join(defines)} for {ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # a long compile says so now and then
    done = threading.Event()

    def ticker() -> None:
        while not done.wait(15.0):
            print(
                f"[fastgen_amd] ... still compiling {src.name} ({time.time() - t0:.0f} s)",
                file=sys.stderr,
                flush=True,
            )

    th = threading.Thread(target=ticker, daemon=True)
    if verbose:
        th.start()
    log, _ = proc.communicate()
    done.set()
    if proc.returncode != 0 or not tmp_out.is_file():
        tmp_out.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed for {src}:\n{' '.join(cmd)}\n{log}")
    os.replace(tmp_out, out)
    # libraries of older sources are of no use any more
    for old in out_dir.glob(f"libfg_{stem}-*.so"):
        if old != out:
            old.unlink(missing_ok=True)
    if verbose:
        print(
            f"[fastgen_amd] built {out.name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True
        )
    return out


def build_all(*, force: bool = True, verbose: bool = True, jobs: int = 8) -> Dict[str, Path]:
    """Compile every kernel library (``force``: also those already built)."""
    from concurrent.futures import ThreadPoolExecutor

    every = list(LIBRARIES) + [f"{b}@{v}" for b, (_, _, values) in VARIANT_LIBRARIES.items() for v in values]
    names = [n for n in every if force or find_built(n) is None]
    out = {n: find_built(n) for n in every if n not in names}
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        for n, p in zip(names, ex.map(lambda n: compile_library(n, verbose=verbose), names)):
            out[n] = p
    return out  # type: ignore[return-value]


def load(name: str) -> ctypes.CDLL:
    """The loaded library ``name``; found, or compiled at this first call."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        if name not in LIBRARIES and name.split("@")[0] not in VARIANT_LIBRARIES:
            raise KeyError(f"no kernel library named {name!r}")
        path = find_built(name) or compile_library(name)
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from e
        _loaded[name] = lib
        return lib
