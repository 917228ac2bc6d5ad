"""Builds and loads the HIP kernel libraries (gfx950 only).

There is one core library, ``libjvamd.so``, made of every ``csrc/*.hip`` file, and
one small library per attention head size, ``libjvamd_attn_d<D>.so``, made of
``csrc/specialized/attention_mfma.hip`` with ``-DJV_HEAD_DIM=<D>``: a model
compiles only the head size it has.  Libraries live in ``csrc/_build`` inside the
package (or, if that is not writable, in a per-user folder under the system
temporary directory) next to a stamp of the sources they were built from; a
library whose stamp does not match is rebuilt.  Nothing falls back to another
implementation: if hipcc or the GPU code is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
HIPCC_FLAGS = [
    "-O3",
    f"--offload-arch={ARCH}",
    "-fPIC",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
ATTN_HEAD_DIMS = tuple(range(16, 257, 16))

_lock = threading.Lock()
_handles: dict[str, ctypes.CDLL] = {}


class KernelLibraryError(RuntimeError):
    """The GPU kernel library could not be built or loaded."""


def _say(msg: str) -> None:
    print(f"[jax_vllm_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelLibraryError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


_build_dir: "Path | None" = None
_build_dir_lock = threading.Lock()


def build_dir() -> Path:
    """Where the libraries live: decided once per process (the parallel builds all ask)."""
    global _build_dir
    with _build_dir_lock:
        if _build_dir is None:
            d = CSRC / "_build"
            try:
                d.mkdir(exist_ok=True)
                probe = d / f".w{os.getpid()}"
                probe.write_text("")
                probe.unlink(missing_ok=True)
            except OSError:
                d = Path(tempfile.gettempdir()) / f"jax_vllm_amd_build_{os.getuid()}"
                d.mkdir(parents=True, exist_ok=True)
            _build_dir = d
        return _build_dir


def _core_sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _own_headers(sources: list[Path]) -> list[Path]:
    """The package's headers that these sources include, directly or through one another."""
    found, todo = {}, list(sources)
    while todo:
        src = todo.pop()
        for line in src.read_text().splitlines():
            line = line.strip()
            if line.startswith("#include \""):
                header = (src.parent / line.split("\"")[1]).resolve()
                if header.exists() and header not in found:
                    found[header] = True
                    todo.append(header)
    return sorted(found)


def _stamp(sources: list[Path], extra: str = "") -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(extra.encode())
    for p in sources + _own_headers(sources):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()


def _run(cmd: list[str]) -> None:
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a HOME it can ignore
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        raise KernelLibraryError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}")


def _compile_link(name: str, sources: list[Path], defines: list[str], stamp: str) -> Path:
    out_dir = build_dir()
    hipcc = _hipcc()
    t0 = time.time()
    _say(f"compiling {name} from {len(sources)} source file(s) for {ARCH} ...")
    objs = []

    def one(src: Path) -> Path:
        obj = out_dir / f"{name}.{src.stem}.{os.getpid()}.o"
        _run([hipcc, *HIPCC_FLAGS, *defines, "-I", str(CSRC), "-c", str(src), "-o", str(obj)])
        _say(f"  {src.name} done ({time.time() - t0:.0f}s)")
        return obj

    workers = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as ex:
        objs = list(ex.map(one, sources))
    tmp = out_dir / f"{name}.{os.getpid()}.tmp.so"
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)])
    for o in objs:
        o.unlink(missing_ok=True)
    final = out_dir / f"{name}.so"
    os.replace(tmp, final)  # atomic: a concurrent process sees the old or the new file
    (out_dir / f"{name}.stamp").write_text(stamp)
    _say(f"{name}.so built in {time.time() - t0:.0f}s")
    return final


def _ensure(name: str, sources: list[Path], defines: list[str], force: bool) -> Path:
    stamp = _stamp(sources, " ".join(defines))
    out_dir = build_dir()
    so, st = out_dir / f"{name}.so", out_dir / f"{name}.stamp"
    if not force and so.exists() and st.exists() and st.read_text() == stamp:
        return so
    return _compile_link(name, sources, defines, stamp)


def _attn_source() -> Path:
    return CSRC / "specialized" / "attention_mfma.hip"


def build_all(force: bool = True) -> None:
    """Compile the core library and the attention library of every supported head size."""
    _ensure("libjvamd", _core_sources(), [], force)
    workers = max(1, min(int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as ex:
        list(ex.map(lambda d: _ensure(f"libjvamd_attn_d{d}", [_attn_source()], [f"-DJV_HEAD_DIM={d}"], force),
                    ATTN_HEAD_DIMS))


def _load(name: str, sources: list[Path], defines: list[str]) -> ctypes.CDLL:
    with _lock:
        if name in _handles:
            return _handles[name]
        import torch  # noqa: F401  (its HIP runtime must be the one in the process)

        try:
            so = _ensure(name, sources, defines, force=False)
            lib = ctypes.CDLL(str(so))
        except OSError as e:
            raise KernelLibraryError(f"cannot load {name}: {e}") from e
        _handles[name] = lib
        return lib


def core() -> ctypes.CDLL:
    """The core kernel library (built at first use if missing or stale)."""
    lib = _handles.get("libjvamd")
    return lib if lib is not None else _load("libjvamd", _core_sources(), [])


def attention(head_dim: int) -> ctypes.CDLL:
    """The MFMA attention library specialised for one head size."""
    if head_dim not in ATTN_HEAD_DIMS:
        raise KernelLibraryError(
            f"no MFMA attention kernel for head size {head_dim}: supported are multiples of 16 up to {ATTN_HEAD_DIMS[-1]}"
        )
    name = f"libjvamd_attn_d{head_dim}"
    lib = _handles.get(name)
    return lib if lib is not None else _load(name, [_attn_source()], [f"-DJV_HEAD_DIM={head_dim}"])
