"""Compiles the HIP sources for gfx950 into shared libraries and loads them.

``libli_core.so`` holds every kernel whose sizes are run-time values; the
attention kernels are compiled once per head size (``libli_attn_hd<N>.so``), at
the first call that needs that size.  Libraries are kept beside the sources (or in
a temporary folder when that is not writable) with a stamp of the sources they
were built from, and are rebuilt when the sources change.  There is no other
implementation behind these libraries: without them nothing runs.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
CORE_SOURCES = ("elementwise.hip", "gemm.hip", "gemm_prefill.hip", "sampling.hip")
ATTN_SOURCE = "attention.hip"
# the headers a library's sources include (its stamp covers them)
HEADERS = {"libli_core.so": ("common.h", "gemm_common.h", "no_alloc.h")}
DEFAULT_HEADERS = ("common.h",)
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

_lock = threading.Lock()
_loaded: dict = {}


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[llm_infer_amd] {msg}", file=sys.stderr, flush=True)


def _preferred_dir() -> str:
    return os.environ.get("LLM_INFER_AMD_BUILD_DIR") or os.path.join(CSRC, "_build")


def build_dir() -> str:
    """Where libraries are built: the preferred folder, or one under the temporary folder if that
    cannot be written (a checkout that belongs to someone else)."""
    d = _preferred_dir()
    try:
        os.makedirs(d, exist_ok=True)
        fd, probe = tempfile.mkstemp(prefix=".w", dir=d)       # a name of its own: builds run side by side
        os.close(fd)
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"llm_infer_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels cannot be built and there is no other implementation")


def _stamp(sources, defines, lib_name="") -> str:
    h = hashlib.sha256()
    for name in tuple(sources) + HEADERS.get(lib_name, DEFAULT_HEADERS):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    h.update(" ".join(FLAGS + list(defines)).encode())
    return h.hexdigest()


def _run(cmd, what):
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())            # hipcc wants a home for its temporary files
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{out}")
    return out


# Kernels that count their own loads in flight (waits placed by hand): a register spilled by the compiler
# would be a load that they do not count, so a build in which they use scratch memory is refused.
# (gemm_wreg: W into a ring of registers by global_load_dwordx4; attn_prefill: the fragments of a page out of
# LDS by ds_read_b128; both written as instructions whose results the compiler knows nothing about until the
# hand-counted wait.)
NO_SCRATCH = {"gemm_prefill.hip": "gemm_wreg_kernel", "attention.hip": "attn_prefill_kernel"}


def _check_no_scratch(report: str, kernel: str, src: str) -> None:
    """``report``: the compiler's resource remarks (-Rpass-analysis=kernel-resource-usage)."""
    name, seen = None, 0
    for line in report.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line and name and kernel in name:
            seen += 1
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size != 0:
                raise BuildError(f"{src}: {name} uses {size} bytes of scratch memory a lane; its waits count on none")
    if seen == 0:
        raise BuildError(f"{src}: the compiler reported no resource usage for {kernel}")


def _build_library(lib_name: str, sources, defines=(), force=False) -> str:
    stamp = _stamp(sources, defines, lib_name)
    if not force:
        # a library built from these very sources is taken where it lies, also from a folder that
        # cannot be written
        for d in dict.fromkeys((_preferred_dir(), build_dir())):
            lib = os.path.join(d, lib_name)
            if os.path.isfile(lib) and os.path.isfile(lib + ".stamp"):
                with open(lib + ".stamp") as f:
                    if f.read().strip() == stamp:
                        return lib
    d = build_dir()
    lib = os.path.join(d, lib_name)
    stamp_file = lib + ".stamp"
    hipcc = _hipcc()
    _say(f"compiling {lib_name} for {ARCH} ...")
    t0 = time.time()
    tag = f"{os.getpid()}_{threading.get_ident()}"
    objs = []

    def compile_one(src):
        obj = os.path.join(d, f"{lib_name}.{src}.{tag}.o")
        report = ["-Rpass-analysis=kernel-resource-usage"] if src in NO_SCRATCH else []
        out = _run([hipcc, *FLAGS, *defines, *report, "-c", os.path.join(CSRC, src), "-o", obj], f"{lib_name}:{src}")
        if report:
            _check_no_scratch(out, NO_SCRATCH[src], src)
        return obj
    try:
        with ThreadPoolExecutor(max_workers=min(4, len(sources))) as pool:
            objs = list(pool.map(compile_one, sources))
        tmp = lib + f".{tag}.tmp"
        _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp, *objs], f"{lib_name} (link)")
        os.replace(tmp, lib)
        with open(stamp_file, "w") as f:
            f.write(stamp)
    finally:
        for o in objs:
            if os.path.isfile(o):
                os.remove(o)
    _say(f"built {lib_name} in {time.time() - t0:.0f} s")
    return lib


def _load(lib_name, sources, defines=(), force=False):
    with _lock:
        if not force and lib_name in _loaded:
            return _loaded[lib_name]
        import torch  # noqa: F401  (the HIP runtime must be the one torch has loaded)
        path = _build_library(lib_name, sources, defines, force)
        _loaded[lib_name] = ctypes.CDLL(path)
        return _loaded[lib_name]


def core_library(force=False):
    return _load("libli_core.so", CORE_SOURCES, (), force)


def attention_library(head_dim: int, force=False):
    if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
        raise BuildError(f"head size {head_dim}: the attention kernels take multiples of 16 up to 256")
    return _load(f"libli_attn_hd{head_dim}.so", (ATTN_SOURCE,), (f"-DHEAD_DIM={head_dim}",), force)


def build_all(head_dims=(16, 32, 48, 64, 128), force=True) -> None:
    """Compile the core library and the attention library for each head size given."""
    core_library(force=force)
    with ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(lambda hd: _build_library(f"libli_attn_hd{hd}.so", (ATTN_SOURCE,),
                                                (f"-DHEAD_DIM={hd}",), force), head_dims))
