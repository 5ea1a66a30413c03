"""Builds and loads the HIP libraries, one shared object per source file under `csrc/`.

A library is compiled with hipcc for gfx950 the first time something in it is called and
kept beside the package (`minfer_amd/_lib/`); a hash of its sources decides whether a
built file is still current.  There is no other backend: if a library can neither be
loaded nor built, the call raises.
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
from typing import Dict, List

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "_lib")

# library name -> source file; HEADERS: what each includes (default: common.h).  A `.cpp` source is
# host code only and is built with the host compiler.
LIBRARIES: Dict[str, str] = {
    "host_random": "host_random.cpp",
    "elementwise": "elementwise.hip",
    "gemm_f32": "gemm_f32.hip",
    "gemm_bf16": "gemm_bf16.hip",
    "attn_tokens_f32": "attn_tokens_f32.hip",
    "attn_decode_bf16": "attn_decode_bf16.hip",
    "attn_prefill_bf16": "attn_prefill_bf16.hip",
    "sampling": "sampling.hip",
    "probe": "probe.hip",
}
HEADERS = {"host_random": ["random_normal.h"],
           "elementwise": ["common.h", "random_normal.h"],
           "attn_tokens_f32": ["common.h", "attn_tokens_impl.h"],
           "attn_decode_bf16": ["common.h", "attn_tokens_impl.h", "noalloc.h"]}

HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-shared", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-pthread", "-ffp-contract=off", "-Wno-unknown-pragmas"]


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP "
                           "kernels cannot be built and there is no other backend")


def is_host_library(name: str) -> bool:
    return LIBRARIES[name].endswith(".cpp")


def _host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if cand and (os.path.exists(cand) or shutil.which(cand)):
            return cand
    raise KernelBuildError("no host C++ compiler found (looked at $CXX, g++, c++, clang++)")


def source_hash(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(HOST_FLAGS if is_host_library(name) else HIPCC_FLAGS).encode())
    for fname in [LIBRARIES[name]] + HEADERS.get(name, ["common.h"]):
        with open(os.path.join(CSRC, fname), "rb") as f:
            h.update(fname.encode())
            h.update(f.read())
    return h.hexdigest()


def lib_dir() -> str:
    """Beside the package; a per-user folder under the temporary directory when the package
    folder cannot be written (a read-only checkout)."""
    global LIB_DIR
    try:
        os.makedirs(LIB_DIR, exist_ok=True)
        if os.access(LIB_DIR, os.W_OK):
            return LIB_DIR
    except OSError:
        pass
    import tempfile
    alt = os.path.join(tempfile.gettempdir(), f"minfer_amd_lib_{os.getuid()}")
    os.makedirs(alt, exist_ok=True)
    have = os.path.join(os.path.dirname(CSRC), "_lib")
    if os.path.isdir(have):           # built files that came with the checkout still count
        for f in os.listdir(have):
            if not os.path.exists(os.path.join(alt, f)):
                shutil.copy(os.path.join(have, f), os.path.join(alt, f))
    LIB_DIR = alt
    return LIB_DIR


def lib_path(name: str) -> str:
    return os.path.join(lib_dir(), f"libmf_{name}.so")


def is_current(name: str) -> bool:
    so, stamp = lib_path(name), lib_path(name) + ".hash"
    if not (os.path.exists(so) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_hash(name)


def _say(msg: str) -> None:
    print(f"[minfer_amd] {msg}", file=sys.stderr, flush=True)


def compile_library(name: str, quiet: bool = False) -> str:
    """Compiles one library; prints a line at start and every 15 s while hipcc runs."""
    so = lib_path(name)
    tmp = f"{so}.{os.getpid()}.tmp"
    if is_host_library(name):
        cmd = [_host_compiler()] + HOST_FLAGS + ["-I", CSRC, os.path.join(CSRC, LIBRARIES[name]), "-o", tmp]
    else:
        cmd = [_hipcc()] + HIPCC_FLAGS + ["-I", CSRC, os.path.join(CSRC, LIBRARIES[name]), "-o", tmp]
    if not quiet:
        _say(f"compiling {LIBRARIES[name]}" + ("" if is_host_library(name) else " for gfx950") + " ...")
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("TMPDIR", "/tmp")
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=lib_dir())
    done = threading.Event()

    def ticker():
        while not done.wait(15.0):
            _say(f"  still compiling {LIBRARIES[name]} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    out = proc.communicate()[0].decode(errors="replace")
    done.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        raise KernelBuildError(f"{os.path.basename(cmd[0])} failed on {LIBRARIES[name]}:\n" + "\n".join(lines[-60:]))
    os.replace(tmp, so)
    with open(so + ".hash", "w") as f:
        f.write(source_hash(name))
    if not quiet:
        _say(f"built {os.path.basename(so)} in {time.time() - t0:.1f} s")
    return so


def build_all(force: bool = True, jobs: int = 4) -> List[str]:
    """Compiles every library (always, when `force`), a few at a time."""
    names = [n for n in LIBRARIES if force or not is_current(n)]
    errors, lock = [], threading.Lock()
    pending = list(names)

    def worker():
        while True:
            with lock:
                if not pending:
                    return
                n = pending.pop(0)
            try:
                compile_library(n)
            except Exception as e:  # collected and raised together below
                with lock:
                    errors.append(e)
    threads = [threading.Thread(target=worker) for _ in range(max(1, min(jobs, len(names))))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise KernelBuildError("\n".join(str(e) for e in errors))
    return [lib_path(n) for n in names]


_loaded: Dict[str, ctypes.CDLL] = {}
_load_lock = threading.Lock()


def load(name: str) -> ctypes.CDLL:
    """The loaded library, compiled first if it is missing or its sources changed."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _load_lock:
        if name in _loaded:
            return _loaded[name]
        if name not in LIBRARIES:
            raise KernelBuildError(f"unknown kernel library {name!r}")
        if not is_current(name):
            compile_library(name)
        try:
            lib = ctypes.CDLL(lib_path(name))
        except OSError as e:
            raise KernelBuildError(f"cannot load {lib_path(name)}: {e}") from None
        _loaded[name] = lib
        return lib
