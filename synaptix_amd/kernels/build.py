"""Compile the native sources and load them through ctypes.

Four kinds of library:
  core            every kernel whose sizes are run-time parameters (hipcc, gfx950)
  attn_hd<N>      the bf16 MFMA attention kernels, compiled for one head size (hipcc, gfx950)
  runtime         host code only: cache bookkeeping, step tables, the sampler's random stream
                  (the host C++ compiler)
  ref             host code only: the kernels' plain C++ twins, the oracle of the kernel tests

A library is built at its first use if no built file matches the sources, which is how the
reference treats its kernels too (compiled at first use; crates/synaptix-kernels-cuda/src/kernels/compile.rs).
Built files live in `synaptix_amd/_lib/` when that is writable, else in a per-user temporary folder.
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
# packed 32-bit float instructions are switched off for all device code
FLAGS = ["-O3", f"--offload-arch={ARCH}", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden"]
CORE_SOURCES = ["elementwise.hip", "sampling.hip", "gemm.hip", "attention_f32.hip", "probes.hip"]
RUNTIME_SOURCES = ["runtime.cpp"]
REF_SOURCES = ["ref/ref_kernels.cpp"]          # the kernels' plain C++ twins (host code)
ATTN_SOURCE = "attention_bf16.hip"
HEADERS = ["common.h", "no_alloc.h"]


class KernelBuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[synaptix_amd] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and $ROCM_PATH/bin); "
                           "the kernels of synaptix_amd cannot be built")


def find_host_compiler() -> str:
    for cand in (os.environ.get("CXX"), "g++", "c++", "clang++"):
        path = shutil.which(cand) if cand else None
        if path:
            return path
    return find_hipcc()      # it compiles plain C++ as well


def lib_dirs() -> list:
    """Where built libraries may lie, best first."""
    in_tree = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "_lib")
    tmp = os.path.join(tempfile.gettempdir(), f"synaptix_amd_lib_{os.getuid()}")
    return [in_tree, tmp]


def _writable_dir() -> str:
    for d in lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            with tempfile.NamedTemporaryFile(dir=d, prefix=".probe_"):
                pass
            return d
        except OSError:
            continue
    raise KernelBuildError("no writable folder for the built kernels: " + ", ".join(lib_dirs()))


def _digest(sources, defines) -> str:
    host = list(sources) in (RUNTIME_SOURCES, REF_SOURCES)
    h = hashlib.sha256()
    for name in list(sources) + ([] if host else HEADERS):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join((HOST_FLAGS if host else FLAGS) + list(defines)).encode())
    return h.hexdigest()[:16]


def _spec(name: str):
    if name == "runtime":
        return RUNTIME_SOURCES, []
    if name == "ref":
        return REF_SOURCES, []
    if name == "core":
        return CORE_SOURCES, []
    if name.startswith("attn_hd"):
        hd = int(name[len("attn_hd"):])
        if hd % 16 != 0 or not (16 <= hd <= 256):
            raise KernelBuildError(f"bf16 attention kernels exist for head sizes 16, 32, ..., 256; got {hd}")
        return [ATTN_SOURCE], [f"-DSYN_HD={hd}"]
    raise KernelBuildError(f"unknown kernel library {name!r}")


def _find_built(name: str, digest: str):
    for d in lib_dirs():
        so = os.path.join(d, f"libsynaptix_{name}.so")
        tag = so + ".digest"
        try:
            with open(tag) as f:
                if f.read().strip() == digest and os.path.isfile(so):
                    return so
        except OSError:
            pass
    return None


def compile_library(name: str, quiet: bool = False) -> str:
    """Compile `name` unconditionally; return the path of the built file."""
    sources, defines = _spec(name)
    digest = _digest(sources, defines)
    out_dir = _writable_dir()
    so = os.path.join(out_dir, f"libsynaptix_{name}.so")
    tmp_so = f"{so}.{os.getpid()}.tmp"
    paths = [os.path.join(CSRC, s) for s in sources]
    if name in ("runtime", "ref"):
        cmd = [find_host_compiler()] + HOST_FLAGS + paths + ["-o", tmp_so]
    else:
        cmd = [find_hipcc()] + FLAGS + defines + paths + ["-o", tmp_so]
    if not quiet:
        target = "the host" if name in ("runtime", "ref") else ARCH
        _say(f"compiling {os.path.basename(so)} for {target} ({len(sources)} source file(s)) ...")
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=out_dir)
    done = threading.Event()

    def ticker():
        while not done.wait(10.0):
            _say(f"  still compiling {os.path.basename(so)} ({time.time() - t0:.0f} s)")

    th = threading.Thread(target=ticker, daemon=True)
    if not quiet:
        th.start()
    log, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        try:
            os.remove(tmp_so)
        except OSError:
            pass
        raise KernelBuildError(f"{os.path.basename(cmd[0])} failed for {name} (exit {proc.returncode}):\n{log}")
    os.replace(tmp_so, so)
    with open(so + ".digest", "w") as f:
        f.write(digest)
    if not quiet:
        _say(f"built {os.path.basename(so)} in {time.time() - t0:.1f} s")
    return so


_LOADED: dict = {}
_LOCK = threading.Lock()


def load_library(name: str) -> ctypes.CDLL:
    """The built library `name`, compiled first if no built file matches the sources."""
    with _LOCK:
        if name in _LOADED:
            return _LOADED[name]
        sources, defines = _spec(name)
        so = _find_built(name, _digest(sources, defines))
        if so is None:
            so = compile_library(name)
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise KernelBuildError(f"cannot load {so}: {e}") from None
        if name == "runtime":
            lib.syn_rt_last_error.restype = ctypes.c_char_p
        elif name == "ref":
            pass            # the twins check nothing and report nothing: their callers are tests
        else:
            lib.syn_last_error.restype = ctypes.c_char_p
        _LOADED[name] = lib
        return lib


def build_all(head_dims=(16, 32, 64, 128)) -> list:
    """Compile the runtime, the core library and the attention library of each head size, in parallel."""
    names = ["runtime", "ref", "core"] + [f"attn_hd{h}" for h in head_dims]
    results, errors = {}, []

    def work(n):
        try:
            results[n] = compile_library(n)
        except Exception as e:  # collected and raised below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    return [results[n] for n in names]
