"""Builds the native libraries in-tree: the HIP kernel modules for gfx950 with hipcc, and the
host-side runtime (plain C++, no device code) with the host compiler.

Sources live in ``photon_infer_amd/csrc``; each *module* is a handful of files linked into
``csrc/_build/libphoton_<module>.so``.  A module is compiled when first needed (or when its
sources changed since the library was built), one compiler process per file in parallel,
with a progress line every few seconds on stderr.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List

from ..errors import KernelLibraryMissing

CSRC_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

# module -> sources.  "core" holds every kernel the float32 path needs; "bf16" adds the
# matrix-core kernels that only the bfloat16 path uses.
MODULES: Dict[str, List[str]] = {
    "core": ["elementwise.hip", "gemm_general.hip", "attention_general.hip", "sampling.hip"],
    "bf16": ["gemm_mfma.hip", "gemm_skinny.hip", "attention_mfma.hip", "attention_decode.hip"],
    # host only: cache manager bookkeeping (needs no GPU and no hipcc)
    "runtime": ["runtime/cache.cpp"],
    # host only: the engine for C / C++ programs (hosts an interpreter; links libpython)
    "api": ["api/photon_engine.cpp"],
}
HEADERS = ["common.h", "mfma.h", "addressing.h", "attention_mfma.h", "sampling.h"]
HOST_MODULES = {"runtime", "api"}
HOST_HEADERS = {"api": ["api/photon_engine.h"]}
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]


def sanitize_flags() -> List[str]:
    """Compiler and linker flags for the host modules from ``PHOTON_SANITIZE`` (for instance
    ``address,undefined``): the libraries are then built beside the ordinary ones, as
    ``libphoton_<module>.<sanitizers>.so``.  A program that loads an address-sanitized library
    must itself start under that sanitizer's runtime; ``build_host_program`` builds such programs
    whole.  Device code is never built with sanitizers."""
    names = os.environ.get("PHOTON_SANITIZE", "").strip()
    if not names:
        return []
    return [f"-fsanitize={names}", "-fno-omit-frame-pointer", "-fno-sanitize-recover=all", "-g", "-O1"]


def build_host_program(sources: List[str], out_path: str, sanitize: str = "", extra_flags: List[str] = ()) -> str:
    """Compile host-only C++ sources (absolute paths, or names under csrc/) into the program
    ``out_path``, optionally under sanitizers (``sanitize="address,undefined"``)."""
    flags = [f for f in HOST_FLAGS if f != "-fPIC"]
    if sanitize:
        flags += [f"-fsanitize={sanitize}", "-fno-omit-frame-pointer", "-fno-sanitize-recover=all", "-g", "-O1"]
    paths = [s if os.path.isabs(s) else os.path.join(CSRC_DIR, s) for s in sources]
    _run([_host_compiler(), *flags, *extra_flags, "-I", CSRC_DIR, *paths, "-o", out_path], os.path.basename(out_path))
    return out_path

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed float32 instructions off for device code (the host pass does not know the feature)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]
# Per file: the prompt-attention kernel keeps its matrix-core accumulators in ordinary vector
# registers.  In the accumulator registers the allocator moved them between register tuples
# from one matrix instruction to the next (hundreds of copies per 32 keys at head size 128).
FILE_FLAGS: Dict[str, List[str]] = {
    "attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def _log(msg: str) -> None:
    print(f"[photon_infer_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelLibraryMissing("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                               "the kernels cannot be built and there is no fallback")


def _host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/lib/llvm/bin/clang++"):
        if cand and (os.path.isfile(cand) or shutil.which(cand)):
            return cand
    raise KernelLibraryMissing("no C++ compiler was found (looked at $CXX, g++, c++, clang++); "
                               "the runtime library cannot be built")


def python_embed_flags():
    """(compile flags, link flags) for a program or library that hosts this interpreter."""
    import sysconfig
    inc = sysconfig.get_paths()["include"]
    libdir = sysconfig.get_config_var("LIBDIR") or "/usr/lib"
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_python_version()
    return [f"-I{inc}"], [f"-L{libdir}", f"-Wl,-rpath,{libdir}", f"-lpython{version}", "-ldl"]


def _build_dir() -> str:
    d = os.path.join(CSRC_DIR, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"photon_infer_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def source_hash(module: str) -> str:
    host = module in HOST_MODULES
    h = hashlib.sha256(" ".join(HOST_FLAGS + sanitize_flags() if host else HIPCC_FLAGS).encode())
    for name in MODULES[module] + (HOST_HEADERS.get(module, []) if host else HEADERS):
        h.update(" ".join(FILE_FLAGS.get(name, [])).encode())
        path = os.path.join(CSRC_DIR, name)
        if os.path.isfile(path):
            with open(path, "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def library_path(module: str) -> str:
    tag = os.environ.get("PHOTON_SANITIZE", "").strip().replace(",", "-") if module in HOST_MODULES else ""
    return os.path.join(_build_dir(), f"libphoton_{module}{'.' + tag if tag else ''}.so")


def is_current(module: str) -> bool:
    lib = library_path(module)
    stamp = lib + ".hash"
    if not (os.path.isfile(lib) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_hash(module)


def _run(cmd: List[str], what: str) -> None:
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a HOME for its caches
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        raise KernelLibraryMissing(f"building {what} failed (exit {proc.returncode}):\n{' '.join(cmd)}\n{proc.stdout}")
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l).strip()
    if out:
        _log(f"{what}: compiler output:\n{out}")


def build_module(module: str, force: bool = False, quiet: bool = False) -> str:
    """Compile and link one module if it is missing or stale; returns the library path."""
    if module not in MODULES:
        raise KernelLibraryMissing(f"unknown kernel module '{module}'")
    lib = library_path(module)
    if not force and is_current(module):
        return lib
    host = module in HOST_MODULES
    hipcc = _host_compiler() if host else _hipcc()
    compile_flags = HOST_FLAGS + sanitize_flags() if host else HIPCC_FLAGS
    link_flags = ["-shared", "-fPIC"] + sanitize_flags() if host else [f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc"]
    link_libs: List[str] = []
    if module == "api":
        compile_flags = compile_flags + python_embed_flags()[0]
        link_libs = python_embed_flags()[1]
    bdir = _build_dir()
    sources = MODULES[module]
    missing = [s for s in sources if not os.path.isfile(os.path.join(CSRC_DIR, s))]
    if missing:
        raise KernelLibraryMissing(f"kernel sources missing for module '{module}': {missing}")
    t0 = time.time()
    if not quiet:
        _log(f"building module '{module}' for {'the host' if host else ARCH} ({len(sources)} files) ...")
    done = threading.Event()

    def heartbeat():
        while not done.wait(10.0):
            _log(f"  still compiling '{module}' ({time.time() - t0:.0f} s)")

    hb = threading.Thread(target=heartbeat, daemon=True)
    if not quiet:
        hb.start()
    objs = []
    try:
        def compile_one(src: str) -> str:
            obj = os.path.join(bdir, f"{module}_{os.path.splitext(os.path.basename(src))[0]}.{os.getpid()}.o")
            base = [hipcc, *compile_flags, "-I", CSRC_DIR, "-c", os.path.join(CSRC_DIR, src), "-o", obj]
            extra = [] if host else FILE_FLAGS.get(src, [])
            try:
                _run(base + extra, src)
            except KernelLibraryMissing:
                if not extra:
                    raise
                _log(f"  {src}: the compiler refused {' '.join(extra)}; compiling without (slower kernel, same results)")
                _run(base, src)
            if not quiet:
                _log(f"  compiled {src} ({time.time() - t0:.0f} s)")
            return obj

        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            objs = list(pool.map(compile_one, sources))
        tmp = f"{lib}.{os.getpid()}.tmp"
        _run([hipcc, *link_flags, *objs, *link_libs, "-o", tmp], f"libphoton_{module}.so")
        os.replace(tmp, lib)
        with open(lib + ".hash", "w") as f:
            f.write(source_hash(module))
    finally:
        done.set()
        for o in objs:
            try:
                os.remove(o)
            except OSError:
                pass
    if not quiet:
        _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def build_all(force: bool = True) -> List[str]:
    return [build_module(m, force=force) for m in MODULES if MODULES[m]]
