"""Compile the HIP sources under ``csrc/`` for gfx950 into shared libraries and load them.

Each library is named after a hash of its sources and flags, so a stale build is never
loaded: a changed source simply asks for a library that is not there yet, which is then
compiled (seconds per file).  Libraries are plain C ABI (``extern "C"``) and are called
through ``ctypes`` with raw device pointers and the caller's HIP stream; they allocate
nothing.

Two kinds of library exist:

* ``core``: every kernel whose code does not depend on the head size.
* ``attn_d<D>``: the matrix-core attention kernels, compiled for one head size ``D``.
  A model compiles only the head sizes it has.

There is no other implementation behind these: if ``hipcc`` is missing or a compile
fails, loading raises.
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

CORE_SOURCES = (
    "elementwise.hip",
    "gemm_f32.hip",
    "attention_generic.hip",
    "sampling.hip",
    "gemm_bf16.hip",
    "gemm_rows.hip",
)
ATTENTION_SOURCES = ("attention_mfma.hip", "attention_f32.hip")
HEADERS = ("common.h", "static_entry.h")

# head sizes built ahead of time by build_all(): every one the kernels take.  A fresh
# checkout compiles only the head size of the model it is asked to run.
DEFAULT_HEAD_DIMS = tuple(range(16, 257, 16))

_HIPCC_FLAGS = (
    "-O3",
    f"--offload-arch={ARCH}",
    "-fPIC",
    "-std=c++17",
    "-Wno-unused-result",
    # packed float32 instructions are kept out of generated code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
)


class KernelBuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[rapid_llm_amd] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise KernelBuildError(
        "hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); the HIP "
        "kernels cannot be compiled and there is no other implementation to fall back to"
    )


def build_dir() -> Path:
    """In-tree ``csrc/_build`` when writable, else a per-user folder under the temp dir."""
    override = os.environ.get("RAPID_LLM_AMD_BUILD_DIR")
    if override:
        path = Path(override)
        path.mkdir(parents=True, exist_ok=True)
        return path
    path = CSRC / "_build"
    try:
        path.mkdir(parents=True, exist_ok=True)
        with tempfile.NamedTemporaryFile(dir=path, prefix=".probe-"):
            pass
        return path
    except OSError:
        path = Path(tempfile.gettempdir()) / f"rapid_llm_amd-build-{os.getuid()}"
        path.mkdir(parents=True, exist_ok=True)
        return path


def _digest(sources: tuple[str, ...], defines: tuple[str, ...]) -> str:
    h = hashlib.sha256()
    for name in sorted(HEADERS) + list(sources):
        h.update(name.encode())
        h.update((CSRC / name).read_bytes())
    h.update(" ".join(_HIPCC_FLAGS + defines).encode())
    return h.hexdigest()[:16]


def library_file(name: str, sources: tuple[str, ...], defines: tuple[str, ...] = ()) -> str:
    return f"librl_{name}-{_digest(sources, defines)}.so"


def _find_built(filename: str) -> Path | None:
    candidates = [CSRC / "_build" / filename]
    override = os.environ.get("RAPID_LLM_AMD_BUILD_DIR")
    if override:
        candidates.insert(0, Path(override) / filename)
    candidates.append(Path(tempfile.gettempdir()) / f"rapid_llm_amd-build-{os.getuid()}" / filename)
    for c in candidates:
        if c.is_file():
            return c
    return None


def _run(cmd: list[str], what: str) -> None:
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME"):
        env["HOME"] = tempfile.gettempdir()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        lines = [
            ln
            for ln in proc.stdout.splitlines()
            if "not a recognized feature for this target" not in ln
        ]
        raise KernelBuildError(f"{what} failed (exit {proc.returncode}):\n" + "\n".join(lines[-60:]))


def compile_library(
    name: str, sources: tuple[str, ...], defines: tuple[str, ...] = (), *, force: bool = False
) -> Path:
    """Compile ``sources`` into one shared library; returns its path."""
    filename = library_file(name, sources, defines)
    if not force:
        built = _find_built(filename)
        if built is not None:
            return built
    hipcc = find_hipcc()
    out_dir = build_dir()
    target = out_dir / filename
    _say(f"compiling {name} ({len(sources)} file(s)) for {ARCH} -> {target}")
    started = time.time()
    done = threading.Event()

    def _heartbeat() -> None:
        while not done.wait(15.0):
            _say(f"  still compiling {name} ({time.time() - started:.0f} s)")

    beat = threading.Thread(target=_heartbeat, daemon=True)
    beat.start()
    try:
        with tempfile.TemporaryDirectory(dir=out_dir, prefix=f".{name}-") as tmp:
            objs = []

            def _one(src: str) -> str:
                obj = os.path.join(tmp, src.replace(".hip", ".o"))
                cmd = [hipcc, *_HIPCC_FLAGS, *defines, f"-I{CSRC}", "-c", str(CSRC / src), "-o", obj]
                _run(cmd, f"hipcc -c {src}")
                return obj

            workers = max(1, min(len(sources), os.cpu_count() or 1, 8))
            with ThreadPoolExecutor(workers) as pool:
                objs = list(pool.map(_one, sources))
            partial = os.path.join(tmp, filename)
            _run(
                [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", partial],
                f"linking {filename}",
            )
            os.replace(partial, target)  # atomic: a concurrent process sees all or nothing
    finally:
        done.set()
    # drop older builds of the same library
    for old in out_dir.glob(f"librl_{name}-*.so"):
        if old.name != filename:
            try:
                old.unlink()
            except OSError:
                pass
    _say(f"built {filename} in {time.time() - started:.1f} s")
    return target


def core_library(force: bool = False) -> Path:
    return compile_library("core", CORE_SOURCES, force=force)


def attention_library(head_dim: int, force: bool = False) -> Path:
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelBuildError(
            f"the matrix-core attention kernels take head sizes in steps of 16 up to 256, "
            f"got {head_dim}"
        )
    # matrix instructions take their accumulators from ordinary vector registers: the softmax
    # rescales them every step, and moving them to and from accumulation registers costs more
    # vector instructions than the rescale itself
    flags = (f"-DRL_HEAD_DIM={head_dim}", "-mllvm", "-amdgpu-mfma-vgpr-form=1")
    return compile_library(f"attn_d{head_dim}", ATTENTION_SOURCES, flags, force=force)


def build_all(head_dims: tuple[int, ...] = DEFAULT_HEAD_DIMS, force: bool = True) -> list[Path]:
    """Compile every library (what ``__graft_entry__.build`` calls)."""
    out = [core_library(force=force)]
    if not all((CSRC / s).is_file() for s in ATTENTION_SOURCES):
        return out
    with ThreadPoolExecutor(min(8, len(head_dims))) as pool:
        out += list(pool.map(lambda d: attention_library(d, force=force), head_dims))
    return out


_LOADED: dict[str, ctypes.CDLL] = {}
_LOCK = threading.Lock()


def load(path: Path) -> ctypes.CDLL:
    # torch must be imported first: its bundled HIP runtime is the one the process uses,
    # and the library's own reference to the runtime then resolves to it
    import torch  # noqa: F401

    key = str(path)
    with _LOCK:
        lib = _LOADED.get(key)
        if lib is None:
            lib = ctypes.CDLL(key)
            _LOADED[key] = lib
        return lib
