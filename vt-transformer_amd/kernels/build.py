"""Compiling the HIP sources for gfx950 and loading the libraries.

Each library is one source file compiled by hipcc into a shared object whose
name carries a hash of the source text, its headers and the flags, so a
changed source never loads a stale build.  Libraries are built in the
package's `_build/` folder; if that is not writable, in a per-user folder
under the system's temporary directory.  Nothing here needs a GPU: hipcc
cross-compiles.

There is no fallback: if a library cannot be built or loaded, the error says
so and the engine does not run.
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
from typing import Dict, Iterable, List, Optional, Tuple

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# libraries that every model needs; attention for the 16-bit types is built per head size
BASE_LIBS = ["vt_elementwise", "vt_gemm_f32", "vt_gemm_bf16", "vt_attn_f32", "vt_sampling"]
DEFAULT_HEAD_DIMS = list(range(16, 257, 16))
# The libraries that handle 16-bit values are built once for bfloat16 and once for float16 (-DVT_LOWP_F16: the same
# sources with the other conversion and the other matrix instruction); the float16 build's name ends in _f16.
HALF_LIBS = ("vt_elementwise", "vt_gemm_bf16", "vt_attn_bf16")


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


_build_dir_cache: Optional[str] = None
_build_dir_lock = threading.Lock()


def _build_dir() -> str:
    global _build_dir_cache
    with _build_dir_lock:
        if _build_dir_cache is None:
            d = os.path.join(os.path.dirname(CSRC), "_build")
            try:
                os.makedirs(d, exist_ok=True)
                fd, probe = tempfile.mkstemp(prefix=".w", dir=d)
                os.close(fd)
                os.remove(probe)
            except OSError:
                d = os.path.join(tempfile.gettempdir(), f"vt_transformer_amd_build_{os.getuid()}")
                os.makedirs(d, exist_ok=True)
            _build_dir_cache = d
        return _build_dir_cache


def _source_hash(src: str, defines: Dict[str, str]) -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith(".h") or name == os.path.basename(src):
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(name.encode())
                h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(defines.items())).encode())
    return h.hexdigest()[:16]


def lib_spec(name: str, head_dim: Optional[int] = None, half: bool = False) -> Tuple[str, str, Dict[str, str]]:
    """(library name, source path, defines).  half: the build whose 16-bit type is float16 (for the libraries that
    have one; the others are the same either way)."""
    half = half and name in HALF_LIBS
    defines: Dict[str, str] = {"VT_LOWP_F16": "1"} if half else {}
    suffix = "_f16" if half else ""
    if name == "vt_attn_bf16":
        if head_dim is None:
            raise ValueError("vt_attn_bf16 is built per head size")
        defines["VT_HEAD_DIM"] = str(head_dim)
        return f"vt_attn_bf16_d{head_dim}{suffix}", os.path.join(CSRC, "vt_attn_bf16.hip"), defines
    return name + suffix, os.path.join(CSRC, name + ".hip"), defines


def lib_path(name: str, head_dim: Optional[int] = None, half: bool = False) -> str:
    lname, src, defines = lib_spec(name, head_dim, half)
    return os.path.join(_build_dir(), f"lib{lname}-{_source_hash(src, defines)}.so")


def compile_lib(name: str, head_dim: Optional[int] = None, force: bool = False, verbose: bool = True,
                half: bool = False) -> str:
    lname, src, defines = lib_spec(name, head_dim, half)
    out = lib_path(name, head_dim, half)
    if os.path.isfile(out) and not force:
        return out
    if not os.path.isfile(src):
        raise KernelBuildError(f"kernel source {src} is missing")
    cmd = [_hipcc()] + FLAGS + [f"-D{k}={v}" for k, v in defines.items()] + ["-I", CSRC, src, "-o"]
    tmp = f"{out}.{os.getpid()}.{threading.get_ident()}.tmp"
    t0 = time.time()
    if verbose:
        print(f"[vt_transformer_amd] compiling {lname} for {ARCH} ...", file=sys.stderr, flush=True)
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd + [tmp], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    # a line now and then while the compiler works
    lines: List[str] = []
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            if verbose:
                print(f"[vt_transformer_amd] still compiling {lname} ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    try:
        text, _ = proc.communicate()
    finally:
        done.set()
    lines = [ln for ln in text.splitlines() if "packed-fp32-ops" not in ln]
    if proc.returncode != 0 or not os.path.isfile(tmp):
        try:
            os.remove(tmp)
        except OSError:
            pass
        raise KernelBuildError(f"hipcc failed for {lname} (exit {proc.returncode}):\n" + "\n".join(lines[-40:]))
    os.replace(tmp, out)
    # drop older builds of the same library
    prefix = f"lib{lname}-"
    for f in os.listdir(os.path.dirname(out)):
        if f.startswith(prefix) and f.endswith(".so") and os.path.join(os.path.dirname(out), f) != out:
            try:
                os.remove(os.path.join(os.path.dirname(out), f))
            except OSError:
                pass
    if verbose:
        print(f"[vt_transformer_amd] built {os.path.basename(out)} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def build_all(head_dims: Iterable[int] = DEFAULT_HEAD_DIMS, force: bool = True, jobs: int = 8, verbose: bool = True) -> List[str]:
    """Compile every library (used by the build check); returns their paths."""
    head_dims = list(head_dims)
    tasks = [(n, None, False) for n in BASE_LIBS] + [("vt_attn_bf16", d, False) for d in head_dims]
    tasks += [(n, None, True) for n in BASE_LIBS if n in HALF_LIBS] + [("vt_attn_bf16", d, True) for d in head_dims]
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, 16))) as ex:
        return list(ex.map(lambda t: compile_lib(t[0], t[1], force=force, verbose=verbose, half=t[2]), tasks))


_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def load_lib(name: str, head_dim: Optional[int] = None, half: bool = False) -> ctypes.CDLL:
    """Load a library, compiling it first if no build of the current source exists.  half: its float16 build."""
    key = lib_spec(name, head_dim, half)[0]
    with _lock:
        if key in _loaded:
            return _loaded[key]
        path = compile_lib(name, head_dim, half=half)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from None
        lib.vt_last_error.restype = ctypes.c_char_p
        _loaded[key] = lib
        return lib
