"""Compiling the native libraries, in-tree, at first use.

Two kinds of library are built from `axon_amd/csrc`:

* `libaxon_kernels_<dtype>.so`: the HIP kernels for gfx950, one build per compute dtype
  (`bfloat16`, `float32`), compiled with hipcc.  A call that needs a dtype compiles that
  dtype only.
* `libaxon_host.so`: the host runtime (cache manager, scheduler), plain C++.

Built files live in `axon_amd/_built/` when that can be written, else in a per-user folder
under the temporary directory.  A stamp beside each library holds a hash of its sources and
flags: a library is reused while the stamp matches and rebuilt when a source changed.
There is no fallback: without a compiler and without a built library, loading fails.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"

KERNEL_SOURCES = ["elementwise.hip", "gemm.hip", "gemm_mfma.hip", "attention.hip", "attention_mfma.hip",
                  "sampling.hip"]
HOST_SOURCES = ["host/cache.cpp", "host/scheduler.cpp", "host/sampler.cpp"]

# Packed 32-bit float instructions are switched off for all device code.  No contraction of a
# product and a sum into a multiply-add unless the source writes one (fmaf): two kernels that
# hold the same expression must round it the same way, whatever surrounds it (hipcc would
# otherwise fuse where a product happens to be in a register and not where it was loaded).
HIP_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-ffp-contract=off", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-Wno-unused-result", "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]

DTYPE_FLAG = {"bfloat16": "-DAXON_BF16=1", "float32": "-DAXON_BF16=0"}


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[axon_amd build] {msg}", file=sys.stderr, flush=True)


def built_dir() -> str:
    """Where libraries are kept: in the package if it can be written, else a per-user folder."""
    override = os.environ.get("AXON_BUILD_DIR")
    if override:
        os.makedirs(override, exist_ok=True)
        return override
    pkg = os.path.join(os.path.dirname(CSRC), "_built")
    try:
        os.makedirs(pkg, exist_ok=True)
        probe = os.path.join(pkg, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return pkg
    except OSError:
        alt = os.path.join(tempfile.gettempdir(), f"axon_amd_built_{os.getuid()}")
        os.makedirs(alt, exist_ok=True)
        return alt


def _existing(sources: List[str]) -> List[str]:
    return [s for s in sources if os.path.exists(os.path.join(CSRC, s))]


def _stamp(sources: List[str], flags: List[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(flags).encode())
    names = sorted(set(_existing(sources)) | {f for f in os.listdir(CSRC) if f.endswith(".h")}
                   | {os.path.join("host", f) for f in os.listdir(os.path.join(CSRC, "host")) if f.endswith(".h")})
    for s in names:
        h.update(s.encode())
        with open(os.path.join(CSRC, s), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _find(tool: str, extra: List[str]) -> str:
    for cand in [shutil.which(tool)] + extra:
        if cand and os.path.exists(cand):
            return cand
    raise BuildError(f"{tool} was not found: the native library cannot be built")


def _run(cmd: List[str], what: str) -> None:
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # compilers want somewhere to keep caches
    p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    t0 = time.time()
    while True:
        try:
            out, _ = p.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")
    if p.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{out}")


def _build(lib_name: str, sources: List[str], compiler: str, flags: List[str], link_flags: List[str], force: bool) -> str:
    out_dir = built_dir()
    lib = os.path.join(out_dir, lib_name)
    stamp_file = lib + ".stamp"
    sources = _existing(sources)
    stamp = _stamp(sources, flags)
    if not force and os.path.exists(lib) and os.path.exists(stamp_file):
        with open(stamp_file) as f:
            if f.read().strip() == stamp:
                return lib
    _say(f"compiling {lib_name} from {len(sources)} sources into {out_dir}")
    obj_dir = os.path.join(out_dir, "obj_" + lib_name.replace(".so", ""))
    os.makedirs(obj_dir, exist_ok=True)
    objs = []

    def one(src: str) -> str:
        obj = os.path.join(obj_dir, src.replace("/", "_") + ".o")
        _run([compiler] + flags + ["-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj], f"{lib_name}: {src}")
        return obj

    workers = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(one, sources))
    tmp = lib + f".tmp{os.getpid()}"
    _run([compiler] + link_flags + ["-shared", "-o", tmp] + objs, f"{lib_name}: link")
    os.replace(tmp, lib)
    with open(stamp_file, "w") as f:
        f.write(stamp)
    _say(f"built {lib_name}")
    return lib


def build_kernels(dtype: str, force: bool = False) -> str:
    """The kernel library of one compute dtype; compiled if missing or stale."""
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"]) if force or not _fresh(f"libaxon_kernels_{dtype}.so", KERNEL_SOURCES,
                                                                        HIP_FLAGS + [DTYPE_FLAG[dtype]]) else "hipcc"
    return _build(f"libaxon_kernels_{dtype}.so", KERNEL_SOURCES, hipcc, HIP_FLAGS + [DTYPE_FLAG[dtype]],
                  [f"--offload-arch={ARCH}", "-fPIC"], force)


def build_host(force: bool = False) -> str:
    cxx = "g++"
    if force or not _fresh("libaxon_host.so", HOST_SOURCES, HOST_FLAGS):
        cxx = _find("g++", ["/usr/bin/g++", "/usr/bin/c++"])
    return _build("libaxon_host.so", HOST_SOURCES, cxx, HOST_FLAGS, ["-fPIC"], force)


def _fresh(lib_name: str, sources: List[str], flags: List[str]) -> bool:
    lib = os.path.join(built_dir(), lib_name)
    try:
        with open(lib + ".stamp") as f:
            return os.path.exists(lib) and f.read().strip() == _stamp(_existing(sources), flags)
    except OSError:
        return False


def build_all(force: bool = True) -> List[str]:
    """Everything: the host runtime and both kernel libraries."""
    return [build_host(force), build_kernels("float32", force), build_kernels("bfloat16", force)]
