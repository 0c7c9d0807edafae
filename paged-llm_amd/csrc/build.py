"""Compiles the HIP sources of this folder for gfx950 and loads them through ctypes.

Each ``.hip`` file becomes one shared library (``hipcc -shared``), optionally specialised by
``-D`` definitions (the MFMA attention kernel is compiled per head size).  A library is built
the first time it is asked for and found again afterwards by a name that carries a digest of
its sources and flags, so a stale build is never loaded.  Libraries go to ``_build/`` beside
the sources; if that folder cannot be written they go to a per-user folder under the system's
temporary directory.  No compiler cache under HOME is needed.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# Packed float math is switched off: some of its forms have given wrong results on this hardware.
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]

# name -> (source file, {define: value})
_LIBS: dict[str, ctypes.CDLL] = {}
_LOCK = threading.Lock()


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _digest(source: str, defines: dict) -> str:
    h = hashlib.sha256()
    headers = sorted(os.path.join(CSRC, name) for name in os.listdir(CSRC) if name.endswith(".h"))
    for path in (*headers, os.path.join(CSRC, source)):
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(repr(sorted(defines.items())).encode())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:12]


def _build_dirs() -> list[str]:
    dirs = [os.path.join(CSRC, "_build")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"paged_llm_amd_build_{uid}"))
    return dirs


def library_file_name(source: str, defines: dict | None = None) -> str:
    defines = defines or {}
    stem = os.path.splitext(source)[0]
    tag = "".join(f"_{k.lower()}{v}" for k, v in sorted(defines.items()))
    return f"libpllm_{stem}{tag}_{_digest(source, defines)}.so"


def find_built(source: str, defines: dict | None = None) -> str | None:
    name = library_file_name(source, defines)
    for d in _build_dirs():
        path = os.path.join(d, name)
        if os.path.isfile(path):
            return path
    return None


def compile_library(source: str, defines: dict | None = None, force: bool = False, quiet: bool = False) -> str:
    """Build one library; returns its path.  Prints a line at the start and every 20 s meanwhile."""
    defines = defines or {}
    if not force:
        found = find_built(source, defines)
        if found:
            return found
    name = library_file_name(source, defines)
    last_err = None
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            with tempfile.NamedTemporaryFile(dir=d, prefix=".probe"):
                pass
        except OSError as e:
            last_err = e
            continue
        out = os.path.join(d, name)
        tmp = out + f".tmp{os.getpid()}_{threading.get_ident()}"
        cmd = [_hipcc(), *FLAGS, *[f"-D{k}={v}" for k, v in sorted(defines.items())],
               os.path.join(CSRC, source), "-o", tmp]
        if not quiet:
            print(f"[paged-llm_amd] compiling {source} {defines or ''} for {ARCH} ...", file=sys.stderr, flush=True)
        t0 = time.time()
        env = dict(os.environ)
        env.setdefault("HOME", tempfile.gettempdir())
        proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=d)
        while True:
            try:
                log, _ = proc.communicate(timeout=20)
                break
            except subprocess.TimeoutExpired:
                if not quiet:
                    print(f"[paged-llm_amd] ... still compiling {source} ({time.time() - t0:.0f} s)",
                          file=sys.stderr, flush=True)
        if proc.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            raise BuildError(f"hipcc failed on {source} (exit {proc.returncode}):\n{log.decode(errors='replace')}")
        os.replace(tmp, out)
        # Older builds of the same target (other digests) are stale now.
        prefix = name[: name.rfind("_") + 1]
        for old in os.listdir(d):
            if old.startswith(prefix) and old.endswith(".so") and old != name and len(old) == len(name):
                try:
                    os.remove(os.path.join(d, old))
                except OSError:
                    pass
        if not quiet:
            print(f"[paged-llm_amd] built {name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        return out
    raise BuildError(f"no writable folder for built libraries (tried {_build_dirs()}): {last_err}")


def load_library(source: str, defines: dict | None = None) -> ctypes.CDLL:
    """The library of one source file, compiled at first use."""
    defines = defines or {}
    key = library_file_name(source, defines)
    with _LOCK:
        lib = _LIBS.get(key)
        if lib is None:
            path = compile_library(source, defines)
            lib = ctypes.CDLL(path)
            _LIBS[key] = lib
        return lib


# Sources every model needs, and the specialised ones per head size.
COMMON_SOURCES = ["elementwise.hip", "gemm_generic.hip", "attention_generic.hip", "sampling.hip", "decode_linear.hip",
                  "attention_noalloc.hip", "stream_linear.hip"]
# Head sizes whose attention library a full build makes (others are compiled at first use).
USUAL_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 256)
# ... and those whose attention library with further score terms in its loops (-DSCORE_TERMS=1) it makes as well.
SCORE_TERMS_HEAD_DIMS = (16, 32, 64, 128)


def all_targets() -> list[tuple[str, dict]]:
    """Everything a full build compiles: the common sources plus the usual specialisations."""
    targets: list[tuple[str, dict]] = [(s, {}) for s in COMMON_SOURCES]
    targets += [("attention_mfma.hip", {"HEAD_DIM": d}) for d in USUAL_HEAD_DIMS]
    targets += [("attention_mfma.hip", {"HEAD_DIM": d, "SCORE_TERMS": 1}) for d in SCORE_TERMS_HEAD_DIMS]
    return targets


def build_all(force: bool = True, jobs: int = 8) -> list[str]:
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        return list(pool.map(lambda t: compile_library(t[0], t[1], force=force), all_targets()))
