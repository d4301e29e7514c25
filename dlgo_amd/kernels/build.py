"""Compiling and loading the HIP kernel files under csrc/.

Each kernel file becomes one shared library per set of compile-time sizes (the
attention kernels are specialised by head size), built with hipcc for gfx950 and
loaded with ctypes.  A library's file name carries a hash of its sources and
flags, so a stale build is never loaded.  Nothing here falls back to another
implementation: without hipcc or without the library the caller gets an error.

computerex/dlgo embeds pre-compiled SPIR-V for its shaders
(gpu/csrc/shaders_spirv.h, gpu/shaders/compile.ps1:62-89); here the code
objects are compiled on first use and kept beside the sources.
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
from typing import Dict, Iterable, Sequence, Tuple

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
# packed float32 instructions are switched off for every kernel
FLAGS = ("-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument")

Defines = Tuple[Tuple[str, int], ...]
Variant = Tuple[str, Defines]

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


def _source_hash(module: str, defines: Defines) -> str:
    h = hashlib.sha256()
    names = [module + ".hip"] + sorted(n for n in os.listdir(CSRC) if n.endswith(".h"))
    for name in names:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(repr(FLAGS).encode())
    h.update(repr(tuple(defines)).encode())
    return h.hexdigest()[:12]


def _file_name(module: str, defines: Defines) -> str:
    tag = "".join(f"-{k}{v}" for k, v in defines)
    return f"{module}{tag}-{_source_hash(module, defines)}.so"


def _build_dirs() -> list[str]:
    """Where libraries are looked for, first hit wins; the first writable one is built into."""
    dirs = []
    if os.environ.get("DLGO_AMD_BUILD_DIR"):
        dirs.append(os.environ["DLGO_AMD_BUILD_DIR"])
    dirs.append(os.path.join(CSRC, "_build"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"dlgo_amd_build_{os.getuid()}"))
    return dirs


def _find(module: str, defines: Defines) -> str | None:
    name = _file_name(module, defines)
    for d in _build_dirs():
        p = os.path.join(d, name)
        if os.path.exists(p):
            return p
    return None


def _writable_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError("no writable place for built kernels (set DLGO_AMD_BUILD_DIR)")


def _say(text: str) -> None:
    print(f"[dlgo_amd] {text}", file=sys.stderr, flush=True)


def ensure_built(variants: Iterable[Variant], force: bool = False, quiet: bool = False) -> None:
    """Compile what is missing of `variants`, several files at a time, and say so now and then."""
    todo = []
    seen = set()
    for module, defines in variants:
        key = (module, tuple(defines))
        if key in seen:
            continue
        seen.add(key)
        if force or _find(module, tuple(defines)) is None:
            todo.append(key)
    if not todo:
        return
    hipcc = _hipcc()
    out_dir = _writable_dir()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())   # the compiler may want a home for its caches
    if not quiet:
        _say(f"compiling {len(todo)} kernel file(s) for {ARCH} into {out_dir}")
    running = []
    t0 = time.time()
    max_jobs = max(1, min(8, (os.cpu_count() or 2)))
    pending = list(todo)
    failures = []
    last_note = time.time()
    while pending or running:
        while pending and len(running) < max_jobs:
            module, defines = pending.pop(0)
            final = os.path.join(out_dir, _file_name(module, defines))
            tmp = final + f".tmp{os.getpid()}"
            cmd = [hipcc, *FLAGS, *[f"-D{k}={v}" for k, v in defines], os.path.join(CSRC, module + ".hip"), "-o", tmp]
            # the compiler's messages go to a file: a pipe that nobody reads while waiting would fill up and stall it
            log_file = open(tmp + ".log", "w+b")
            p = subprocess.Popen(cmd, stdout=log_file, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
            p.log_file = log_file
            running.append((p, module, defines, tmp, final))
        still = []
        for item in running:
            p, module, defines, tmp, final = item
            if p.poll() is None:
                still.append(item)
                continue
            p.log_file.seek(0)
            log = p.log_file.read().decode(errors="replace")
            p.log_file.close()
            try:
                os.remove(tmp + ".log")
            except OSError:
                pass
            if p.returncode != 0 or not os.path.exists(tmp):
                log = "\n".join(l for l in log.splitlines() if "not a recognized feature" not in l)
                failures.append(f"{module} {dict(defines)}:\n{log}")
                if os.path.exists(tmp):
                    os.remove(tmp)
            else:
                os.replace(tmp, final)
                stem = os.path.basename(final).rsplit("-", 1)[0] + "-"
                for other in os.listdir(out_dir):     # builds of older sources of the same variant
                    if other.startswith(stem) and other.endswith(".so") and other != os.path.basename(final) \
                            and len(other) == len(os.path.basename(final)):
                        try:
                            os.remove(os.path.join(out_dir, other))
                        except OSError:
                            pass
                if not quiet:
                    _say(f"built {os.path.basename(final)} ({time.time() - t0:.0f}s)")
                last_note = time.time()
        running = still
        if running:
            time.sleep(0.1)
            if not quiet and time.time() - last_note > 10:
                _say(f"still compiling {', '.join(m for _, m, *_ in running)} ({time.time() - t0:.0f}s)")
                last_note = time.time()
    if failures:
        raise KernelBuildError("hipcc failed:\n" + "\n".join(failures))


def load(module: str, defines: Defines = (), build: bool = True) -> ctypes.CDLL:
    """The loaded library of a kernel file; compiled first if it is not there."""
    defines = tuple(defines)
    key = _file_name(module, defines)
    with _lock:
        if key in _loaded:
            return _loaded[key]
        path = _find(module, defines)
        if path is None:
            if not build:
                raise KernelBuildError(f"kernel library {key} is not built")
            ensure_built([(module, defines)])
            path = _find(module, defines)
            if path is None:
                raise KernelBuildError(f"kernel library {key} missing after build")
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from None
        _loaded[key] = lib
        return lib


def loaded_libraries() -> Sequence[str]:
    return sorted(_loaded)


#: kernel files compiled once per element type (-DDLGO_ELEM=0 float32, 1 bfloat16)
PER_ELEMENT_TYPE = ("gemm", "gemm_rows")
_ELEM_CODE = {"torch.float32": 0, "torch.bfloat16": 1}


def variant(module: str, dtype=None, defines: Defines = ()) -> Variant:
    """The (module, defines) pair of a kernel file for a run dtype."""
    if module in PER_ELEMENT_TYPE:
        if str(dtype) not in _ELEM_CODE:
            raise KernelBuildError(f"{module} is built for float32 or bfloat16, not {dtype}")
        return module, (("DLGO_ELEM", _ELEM_CODE[str(dtype)]),) + tuple(defines)
    return module, tuple(defines)


#: head sizes compiled ahead by build_all(): those of the test configurations and of the benchmark shapes
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 128, 256)


def all_variants(head_dims: Sequence[int] = DEFAULT_HEAD_DIMS) -> list[Variant]:
    out: list[Variant] = [(m, ()) for m in ("embed", "rmsnorm", "rope_kv", "rowwise", "sampling")]
    out += [(m, (("DLGO_ELEM", code),)) for m in ("gemm", "gemm_rows") for code in (0, 1)]
    out += [("attention", (("HEAD_DIM", hd),)) for hd in head_dims]
    return out


def build_all(force: bool = True, quiet: bool = False) -> None:
    ensure_built(all_variants(), force=force, quiet=quiet)
