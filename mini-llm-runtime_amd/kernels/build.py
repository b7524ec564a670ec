"""Compiles the HIP sources under csrc/ for gfx950 and the host sources with the C++
compiler, one shared library per (source, element type), and loads them with ctypes.

A library is built when it is missing or when its sources changed since it was built.  The
libraries live beside the sources (csrc/lib/) when that folder can be written, else in a
per-user folder under the temporary directory.  Several libraries are compiled at once, in
threads, and a progress line goes to stderr every few seconds so that a first call that has
to compile does not look hung.  There is no fallback: a missing compiler or a failed build
raises.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
HIP_FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC"]
# MLR_HOST_SANITIZE=1 in the environment: the host library (page bookkeeping, batch forming) is built with the
# address and undefined-behaviour sanitizers, as its own file, and loaded instead of the plain one.  The
# process must then have the sanitizer's runtime loaded first (LD_PRELOAD=$(gcc -print-file-name=libasan.so)).
# The reference runs its host tests the same way in CI (.github/workflows/ci.yml:60-71).  CPU code only.
HOST_SANITIZE_FLAGS = ["-O1", "-g", "-fno-omit-frame-pointer", "-std=c++17", "-shared", "-fPIC",
                       "-fsanitize=address,undefined", "-fno-sanitize-recover=all"]


def host_sanitized():
    return os.environ.get("MLR_HOST_SANITIZE", "") not in ("", "0")

# name -> (sources relative to csrc/, headers it includes, depends on the element type[, extra link flags])
HIP_LIBRARIES = {
    "elementwise": (["elementwise.hip"], ["common.h"], True),
    "rope_kv": (["rope_kv.hip"], ["common.h"], True),
    "attention": (["attention.hip"], ["common.h"], True),
    "gemm": (["gemm.hip"], ["common.h"], True),
    "attention_tiles": (["attention_tiles.hip"], [], False),      # bfloat16 only by nature
    "sampling": (["sampling.hip"], ["no_alloc.h"], False),
    "library_gemm": (["library_gemm.hip"], [], False, ["-lhipblaslt"]),      # host code around hipBLASLt
}
HOST_LIBRARIES = {
    "host": (["host/cache_manager.cpp", "host/scheduler.cpp"], []),
}

_loaded = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def dtype_tag(dtype):
    import torch
    if dtype == torch.bfloat16:
        return "bf16"
    if dtype == torch.float32:
        return "f32"
    raise BuildError(f"no kernels for element type {dtype}")


def _lib_dir():
    in_tree = os.path.join(CSRC, "lib")
    try:
        os.makedirs(in_tree, exist_ok=True)
        probe = os.path.join(in_tree, f".write_probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return in_tree
    except OSError:
        pass
    base = os.path.join(tempfile.gettempdir(), f"mini_llm_runtime_amd_{os.getuid()}")
    os.makedirs(base, exist_ok=True)
    return base


def _find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH): the HIP kernels "
                     "cannot be built and there is no other path")


def _find_cxx():
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("no C++ compiler found for the host library")


def _plan(name, tag):
    """(output path, command, digest of everything the output depends on)."""
    if name in HOST_LIBRARIES:
        sources, headers = HOST_LIBRARIES[name]
        flags = HOST_SANITIZE_FLAGS if host_sanitized() else HOST_FLAGS
        out = os.path.join(_lib_dir(), f"libmlr_{name}{'_sanitized' if host_sanitized() else ''}.so")
        cmd = [_find_cxx(), *flags, "-o", out] + [os.path.join(CSRC, s) for s in sources]
    else:
        sources, headers, typed, *rest = HIP_LIBRARIES[name]
        link = rest[0] if rest else []
        suffix = f"_{tag}" if typed else ""
        out = os.path.join(_lib_dir(), f"libmlr_{name}{suffix}.so")
        defs = [f"-DMLR_BF16={1 if tag == 'bf16' else 0}"] if typed else []
        cmd = [_find_hipcc(), *HIP_FLAGS, *defs, "-o", out] + [os.path.join(CSRC, s) for s in sources] + link
        flags = HIP_FLAGS + defs + link
    h = hashlib.sha256(" ".join(flags).encode())
    for rel in sources + headers:
        with open(os.path.join(CSRC, rel), "rb") as f:
            h.update(rel.encode())
            h.update(f.read())
    return out, cmd, h.hexdigest()


def _is_current(out, digest):
    stamp = out + ".stamp"
    if not (os.path.isfile(out) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == digest


def _compile(out, cmd, digest):
    tmp = f"{out}.{os.getpid()}.{threading.get_ident()}.tmp"
    cmd = [tmp if c == out else c for c in cmd]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        log = "\n".join(l for l in proc.stdout.splitlines() if "not a recognized feature" not in l)
        raise BuildError(f"build failed: {' '.join(cmd)}\n{log}")
    os.replace(tmp, out)
    with open(out + ".stamp", "w") as f:
        f.write(digest)


def ensure_built(names, dtype=None, force=False, verbose=True):
    """Build every named library that is missing or stale (all of them with force=True)."""
    tag = dtype_tag(dtype) if dtype is not None else None
    todo = []
    for name in names:
        typed = name in HIP_LIBRARIES and HIP_LIBRARIES[name][2]
        if typed and tag is None:
            raise BuildError(f"library {name} needs an element type")
        out, cmd, digest = _plan(name, tag)
        if force or not _is_current(out, digest):
            todo.append((name, out, cmd, digest))
    if not todo:
        return
    errors = []
    done = []

    def work(item):
        try:
            _compile(*item[1:])
        except Exception as err:   # reported below, from the calling thread
            errors.append(err)
        finally:
            done.append(item[0])

    with _lock:
        start = time.time()
        if verbose:
            print(f"[mini-llm-runtime_amd] compiling {len(todo)} kernel librar"
                  f"{'y' if len(todo) == 1 else 'ies'} for {ARCH}: "
                  f"{', '.join(os.path.basename(t[1]) for t in todo)}", file=sys.stderr, flush=True)
        threads = [threading.Thread(target=work, args=(item,)) for item in todo]
        for th in threads:
            th.start()
        while any(th.is_alive() for th in threads):
            for th in threads:
                th.join(timeout=5.0 / max(1, len(threads)))
            if verbose and any(th.is_alive() for th in threads):
                print(f"[mini-llm-runtime_amd] still compiling ({len(done)}/{len(todo)} done, "
                      f"{time.time() - start:.0f} s)", file=sys.stderr, flush=True)
        if verbose:
            print(f"[mini-llm-runtime_amd] compiled in {time.time() - start:.1f} s",
                  file=sys.stderr, flush=True)
    if errors:
        raise errors[0]


def load(name, dtype=None):
    """The ctypes library `name` for element type `dtype`, built first if need be."""
    typed = name in HIP_LIBRARIES and HIP_LIBRARIES[name][2]
    tag = dtype_tag(dtype) if typed else None
    key = (name, tag, host_sanitized() and name in HOST_LIBRARIES)
    if key in _loaded:
        return _loaded[key]
    ensure_built([name], dtype if typed else None)
    out, _, _ = _plan(name, tag)
    try:
        lib = ctypes.CDLL(out)
    except OSError as err:
        raise BuildError(f"cannot load {out}: {err}") from None
    _loaded[key] = lib
    lib._mlr_path = out
    return lib


def build_all(force=True, verbose=True):
    """Every library for both element types (the build check)."""
    import torch
    ensure_built(list(HOST_LIBRARIES), force=force, verbose=verbose)
    untyped = [n for n, v in HIP_LIBRARIES.items() if not v[2]]
    typed = [n for n, v in HIP_LIBRARIES.items() if v[2]]
    ensure_built(untyped, force=force, verbose=verbose)
    for dtype in (torch.float32, torch.bfloat16):
        ensure_built(typed, dtype, force=force, verbose=verbose)
