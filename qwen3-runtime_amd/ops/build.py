"""Compile the HIP sources into shared libraries, in-tree, and find them again.

Two kinds of library of the engine's own: ``core`` (everything whose sizes are
run-time arguments) and ``attn_bf16_d<D>`` (the MFMA attention kernel, one build
per head size). A part defined elsewhere brings its kernels with
``register_library(name, sources)`` and loads them with ``ops.hip.load_library``:
same flags, same cache, same error reporting, no edit here. A library is rebuilt when the hash of its sources and flags changes. The build
is plain ``hipcc`` for gfx950: seconds per file, no Python headers involved, so
a fresh checkout compiles what a model needs at its first call and prints a
line per file while it does.
"""

from __future__ import annotations

import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parents[1]
CSRC = PACKAGE_DIR / "csrc"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    # packed float32 instructions stay off: some of their forms have returned wrong results
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# further hipcc flags (for instance -D switches of a kernel under tuning); part of the libraries' hash
FLAGS += os.environ.get("QWEN3_RUNTIME_AMD_HIPCC_FLAGS", "").split()
CORE_SOURCES = ["runtime.hip", "elementwise.hip", "gemm_f32.hip", "gemm_bf16.hip", "attention_f32.hip", "sampling.hip"]


class BuildError(RuntimeError):
    pass


# libraries registered from outside: name -> (source paths, extra defines)
_REGISTERED: dict[str, tuple[list[Path], list[str]]] = {}


def register_library(name: str, sources, defines=()) -> None:
    """Make ``name`` buildable and loadable: ``sources`` are paths of HIP files (they may
    include ``common.h`` of this package, which is on the include path, and then link
    ``runtime.hip`` for ``qrt_fail`` / ``qrt_last_error`` by listing it as ``"runtime.hip"``).
    Registering the same name with the same sources again is allowed."""
    if name in ("core", "peaks") or name.startswith("attn_bf16_d"):
        raise BuildError(f"{name!r} is a library of the engine's own")
    paths = [CSRC / s if not Path(s).is_absolute() else Path(s) for s in sources]
    for path in paths:
        if not path.is_file():
            raise BuildError(f"library {name!r}: no source file {path}")
    entry = (paths, list(defines))
    if _REGISTERED.get(name, entry) != entry:
        raise BuildError(f"library {name!r} is already registered with other sources")
    _REGISTERED[name] = entry


def registered_libraries() -> list[str]:
    return sorted(_REGISTERED)


def _say(msg: str) -> None:
    print(f"[qwen3_runtime_amd] {msg}", file=sys.stderr, flush=True)


def lib_dir() -> Path:
    """``<package>/_lib`` when it can be written, else a per-user folder under the temp dir."""
    override = os.environ.get("QWEN3_RUNTIME_AMD_LIB_DIR")
    if override:
        path = Path(override)
        path.mkdir(parents=True, exist_ok=True)
        return path
    path = PACKAGE_DIR / "_lib"
    try:
        path.mkdir(exist_ok=True)
        probe = path / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return path
    except OSError:
        path = Path(tempfile.gettempdir()) / f"qwen3_runtime_amd_lib_{os.getuid()}"
        path.mkdir(parents=True, exist_ok=True)
        return path


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def library_spec(name: str) -> tuple[list, list[str]]:
    """Sources (names under ``csrc``, or paths) and extra defines of a library name."""
    if name == "core":
        return CORE_SOURCES, []
    if name == "peaks":  # the device's own bandwidth and MFMA rate, for the measurements
        return ["runtime.hip", "peaks.hip"], []
    if name in _REGISTERED:
        return list(_REGISTERED[name][0]), list(_REGISTERED[name][1])
    if name.startswith("attn_bf16_d"):
        d = int(name[len("attn_bf16_d"):])
        if d % 16 or not 16 <= d <= 512:
            raise BuildError(f"the bfloat16 attention kernel takes head sizes 16..512 in steps of 16, not {d}")
        return ["runtime.hip", "attention_bf16.hip"], [f"-DQRT_HEAD_DIM={d}"]
    raise BuildError(f"unknown library {name!r}; registered from outside: {registered_libraries()}")


def _digest(sources: list, defines: list[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + defines).encode())
    for name in list(sources) + sorted(p.name for p in CSRC.glob("*.h")):
        h.update(Path(name).name.encode())
        h.update((CSRC / name).read_bytes())  # an absolute path stays itself under "/"
    return h.hexdigest()


def library_path(name: str) -> Path:
    return lib_dir() / f"libqrt_{name}.so"


def is_current(name: str) -> bool:
    sources, defines = library_spec(name)
    so = library_path(name)
    stamp = so.with_suffix(".hash")
    return so.exists() and stamp.exists() and stamp.read_text() == _digest(sources, defines)


def _compile_one(hipcc: str, src: Path, obj: Path, defines: list[str]) -> None:
    cmd = [hipcc, *FLAGS, *defines, f"-I{CSRC}", "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")


def build_library(name: str, force: bool = False) -> Path:
    """Compile (if stale or ``force``) and return the library's path."""
    sources, defines = library_spec(name)
    out_dir = lib_dir()
    so = library_path(name)
    stamp = so.with_suffix(".hash")
    digest = _digest(sources, defines)
    with open(out_dir / f".{name}.lock", "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)  # one builder at a time; the others find the result
        if not force and so.exists() and stamp.exists() and stamp.read_text() == digest:
            return so
        hipcc = _hipcc()
        work = out_dir / f"_build_{name}"
        work.mkdir(exist_ok=True)
        t0 = time.time()
        _say(f"compiling {name} for {ARCH}: {len(sources)} files")
        objs = [work / f"{i}_{Path(s).stem}.o" for i, s in enumerate(sources)]

        def one(pair):
            src, obj = pair
            _compile_one(hipcc, CSRC / src, obj, defines)
            _say(f"  {Path(src).name} done ({time.time() - t0:.0f} s)")

        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            list(pool.map(one, zip(sources, objs)))
        tmp = so.with_suffix(f".tmp{os.getpid()}")
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise BuildError(f"linking {so.name} failed:\n{proc.stderr[-4000:]}")
        os.replace(tmp, so)
        stamp.write_text(digest)
        shutil.rmtree(work, ignore_errors=True)
        _say(f"built {so.name} in {time.time() - t0:.0f} s")
    return so


def build_all(head_dims=(16, 32, 48, 64, 80, 96, 112, 128, 256), force: bool = True) -> list[Path]:
    """Every library the tests, the smoke run and the measurements load."""
    names = ["core", "peaks"] + [f"attn_bf16_d{d}" for d in head_dims] + registered_libraries()
    return [build_library(n, force=force) for n in names]
