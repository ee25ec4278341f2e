"""Compiling the native libraries, in-tree, at first use.

Two kinds of library are built from `axon_amd/csrc`:

* `libaxon_kernels_<dtype>.so`: the HIP kernels for gfx950, one build per compute dtype
  (`bfloat16`, `float32`), compiled with hipcc.  A call that needs a dtype compiles that
  dtype only.
* `libaxon_host.so`: the host runtime (cache manager, scheduler), plain C++.
* `libaxon_ext_<name>_<dtype>.so`: one library per kernel source that a part outside the package
  registered (`register_kernel_source`), built like the kernel library, with this package's
  headers on the include path.

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
                  "sampling.hip", "instances.hip", "support.hip"]
# what a library built from a part's own kernel sources gets beside them (the error channel, the
# list of its kernel instances)
EXTENSION_SUPPORT = ["support.hip", "instances.hip"]
HOST_SOURCES = ["host/cache.cpp", "host/scheduler.cpp", "host/sampler.cpp", "host/step.cpp"]

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
    """Sources are named relative to the package's csrc, or by an absolute path."""
    return [s for s in sources if os.path.exists(os.path.join(CSRC, s))]


# --------------------------------------------------------------------------- a part's own kernels
# A part that brings HIP kernels of its own adds files and edits none of this package's:
# `register_kernel_source(path, {entry point: argument types})` names a .hip file anywhere (it may
# include this package's common.h and api.h; its entry points are extern "C", return 0 or a
# negative code after axk_set_error, as the package's own do).  The file is compiled per compute
# dtype into a library of its own, at the first call of one of its entry points
# (`Kernels.call(name, ...)`).
_EXTENSIONS: dict = {}        # absolute path -> {entry point: ctypes argument types}


def register_kernel_source(path: str, signatures: dict) -> None:
    path = os.path.abspath(path)
    if not os.path.isfile(path):
        raise BuildError(f"register_kernel_source: {path} does not exist")
    for other, sigs in _EXTENSIONS.items():
        if other == path:
            continue
        if _stem(other) == _stem(path):       # the library is named after the file
            raise BuildError(f"register_kernel_source: {path} and {other} have the same file name")
        for name in signatures:
            if name in sigs:
                raise BuildError(f"register_kernel_source: {name} is already an entry point of {other}")
    _EXTENSIONS[path] = {name: list(args) for name, args in signatures.items()}


def _stem(path: str) -> str:
    return "".join(c if c.isalnum() else "_" for c in os.path.splitext(os.path.basename(path))[0])


def registered_kernel_sources() -> dict:
    return dict(_EXTENSIONS)


def build_extension(path: str, dtype: str, force: bool = False) -> str:
    """The library of one registered source for one compute dtype; compiled if missing or stale."""
    path = os.path.abspath(path)
    lib_name = f"libaxon_ext_{_stem(path)}_{dtype}.so"
    flags = HIP_FLAGS + [DTYPE_FLAG[dtype]]
    sources = [path] + EXTENSION_SUPPORT
    hipcc = "hipcc" if not force and _fresh(lib_name, sources, flags) else _find("hipcc", ["/opt/rocm/bin/hipcc"])
    return _build(lib_name, sources, hipcc, flags, [f"--offload-arch={ARCH}", "-fPIC"], force)


def _stamp(sources: List[str], flags: List[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(flags).encode())
    names = sorted(set(_existing(sources)) | {f for f in os.listdir(CSRC) if f.endswith(".h")}
                   | {os.path.join("host", f) for f in os.listdir(os.path.join(CSRC, "host")) if f.endswith(".h")})
    for s in names:
        h.update((os.path.basename(s) if os.path.isabs(s) else s).encode())     # a built library travels with the tree
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
        obj = os.path.join(obj_dir, os.path.relpath(os.path.join(CSRC, src), CSRC).replace("/", "_").replace("..", "up") + ".o")
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
