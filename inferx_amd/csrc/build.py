"""Builds the HIP library for gfx950 with hipcc and loads it through ctypes.

The library is plain `extern "C"` entry points over raw device pointers, so it
compiles in seconds per file and needs no Python headers.  It is built in-tree
(`inferx_amd/csrc/_build/libinferx_hip.so`); if that folder cannot be written
the build goes to a per-user folder under the temporary directory.  A loaded
library whose sources have changed since it was built is rebuilt first.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor, as_completed
from typing import List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
LIB_NAME = "libinferx_hip.so"
# packed float32 instructions are switched off for all device code
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes"]

# per source: matrix-core accumulators in ordinary vector registers, where a kernel also rescales them with vector
# instructions between products (the compiler otherwise copies them to and from accumulation registers every time)
FILE_FLAGS = {"attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
              "attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}

# the vendor's library for dense products (csrc/gemm.hip calls its C interface)
LINK_LIBS = ["-lhipblaslt"]

_lib: Optional[ctypes.CDLL] = None


class BuildError(RuntimeError):
    pass


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _digest() -> str:
    h = hashlib.sha256()
    for name in sources() + sorted(f for f in os.listdir(HERE) if f.endswith(".h")):
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + LINK_LIBS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def _say(msg: str) -> None:
    print(f"[inferx_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP library cannot be built")


def _build_dirs() -> List[str]:
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(HERE, "_build"), os.path.join(tempfile.gettempdir(), f"inferx_amd_build_{uid}")]


def _usable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def find_built() -> Optional[str]:
    """Path of a library built from the present sources, if there is one."""
    want = _digest()
    for d in _build_dirs():
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, "digest.txt")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def build(verbose: bool = True) -> str:
    """Compile every .hip source and link the library.  Returns its path."""
    hipcc = _hipcc()
    out_dir = next((d for d in _build_dirs() if _usable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the build: tried " + ", ".join(_build_dirs()))
    srcs = sources()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)  # hipcc wants some HOME; an empty one is fine

    def compile_one(name: str):
        obj = os.path.join(out_dir, name[:-4] + ".o")
        cmd = [hipcc] + FLAGS + FILE_FLAGS.get(name, []) + ["-c", os.path.join(HERE, name), "-o", obj]
        p = subprocess.run(cmd, capture_output=True, text=True, env=env)
        return name, obj, p

    objs = []
    jobs = max(1, min(8, len(srcs), (os.cpu_count() or 2)))
    with ThreadPoolExecutor(jobs) as pool:
        futures = [pool.submit(compile_one, s) for s in srcs]
        for done, fut in enumerate(as_completed(futures), 1):
            name, obj, p = fut.result()
            if p.returncode != 0:
                raise BuildError(f"hipcc failed on {name}:\n{p.stdout}\n{p.stderr}")
            objs.append(obj)
            if verbose:
                _say(f"  [{done}/{len(srcs)}] {name} ({time.time() - t0:.0f}s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    p = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + sorted(objs) + LINK_LIBS,
                       capture_output=True, text=True, env=env)
    if p.returncode != 0:
        raise BuildError(f"hipcc failed to link:\n{p.stdout}\n{p.stderr}")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, "digest.txt"), "w") as f:
        f.write(_digest())
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f}s")
    return lib


# ---- the host library (no GPU code): cache manager, batch layout, scheduler ----------------------------
HOST_DIR = os.path.join(HERE, "host")
HOST_LIB_NAME = "libinferx_host.so"
HOST_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-shared", "-Wall"]
_host_lib: Optional[ctypes.CDLL] = None


def host_sources() -> List[str]:
    return sorted(f for f in os.listdir(HOST_DIR) if f.endswith(".cc"))


def _host_digest() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(HOST_DIR)):
        if name.endswith((".cc", ".h")):
            h.update(name.encode())
            with open(os.path.join(HOST_DIR, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()[:16]


def find_built_host() -> Optional[str]:
    want = _host_digest()
    for d in _build_dirs():
        lib, stamp = os.path.join(d, HOST_LIB_NAME), os.path.join(d, "host_digest.txt")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def build_host(verbose: bool = True) -> str:
    """Compile the host sources with the C++ compiler (g++, else hipcc).  Returns the library's path."""
    cxx = next((c for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"))
                if c and os.path.isfile(c)), None) or _hipcc()
    out_dir = next((d for d in _build_dirs() if _usable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the build: tried " + ", ".join(_build_dirs()))
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    t0 = time.time()
    p = subprocess.run([cxx] + HOST_FLAGS + ["-o", tmp] + [os.path.join(HOST_DIR, s) for s in host_sources()],
                       capture_output=True, text=True)
    if p.returncode != 0:
        raise BuildError(f"{cxx} failed on the host sources:\n{p.stdout}\n{p.stderr}")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, "host_digest.txt"), "w") as f:
        f.write(_host_digest())
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f}s")
    return lib


def load_host() -> ctypes.CDLL:
    """The host library, built first if no current build exists."""
    global _host_lib
    if _host_lib is None:
        path = find_built_host() or build_host()
        try:
            _host_lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from None
    return _host_lib


_C_TYPES = {"int": ctypes.c_int, "int32_t": ctypes.c_int, "int64_t": ctypes.c_int64, "float": ctypes.c_float,
            "double": ctypes.c_double, "size_t": ctypes.c_size_t, "hipStream_t": ctypes.c_void_p}


def signatures() -> dict:
    """name -> (result type, argument types) of every `extern "C"` entry point, read from the sources: with the
    argument types set, ctypes converts plain Python numbers itself (a pointer is an int or None), which costs a
    fraction of building a ctypes object per argument."""
    import re
    out = {}
    for path in sources():
        with open(os.path.join(HERE, path)) as f:
            text = f.read()
        for m in re.finditer(r'extern\s+"C"\s+([\w\s\*]+?)\s*\b(ix_\w+)\s*\(([^)]*)\)\s*\{', text):
            result, name, params = m.group(1).strip(), m.group(2), m.group(3)
            args = []
            for prm in (q.strip() for q in params.split(",")):
                if not prm or prm == "void":
                    continue
                if "*" in prm:
                    args.append(ctypes.c_void_p)
                    continue
                words = [w for w in prm.split() if w != "const"]
                if len(words) != 2 or words[0] not in _C_TYPES:
                    raise BuildError(f"{os.path.basename(path)}: cannot read parameter {prm!r} of {name}")
                args.append(_C_TYPES[words[0]])
            if "*" in result:
                res = ctypes.c_char_p
            elif result in _C_TYPES:
                res = _C_TYPES[result]
            else:
                raise BuildError(f"{os.path.basename(path)}: cannot read result type {result!r} of {name}")
            out[name] = (res, args)
    return out


def load() -> ctypes.CDLL:
    """The library, built first if no current build exists.  Raises if it cannot be had."""
    global _lib
    if _lib is None:
        path = find_built() or build()
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from None
        for name, (res, args) in signatures().items():
            fn = getattr(lib, name)  # every entry point of the sources must be in the library
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib
