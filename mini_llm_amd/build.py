"""Builds the native libraries in-tree and loads them with ctypes.

These live under ``mini_llm_amd/_lib``:

* ``runtime``: the host-only C++ runtime (cache manager, scheduler), built with g++;
* one library per kernel source under ``csrc/kernels`` built with hipcc for gfx950;
* ``engine``: the engine itself (host code that calls the kernel libraries), and the
  program ``mini-llm``, its command line.

A plugin (a shared library that registers further parts and architectures with the engine,
``kind: "plugin"``) is described by its owner with ``register_library`` and built the same way.

A library is rebuilt when the hash of its sources differs from the one recorded
beside it, so a stale binary is never loaded.
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
from typing import Dict, List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "_lib")

GPU_ARCH = "gfx950"
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={GPU_ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 16 dwords of a kernel's arguments arrive in registers with the wavefront instead of
    # being loaded by it: saves the load's latency at the head of every short kernel
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    # MFMA results go to ordinary vector registers, not to the accumulation registers: the kernels here
    # read every result with vector instructions (softmax, epilogues), and each such read or write of an
    # accumulation register is a move of its own (12 % of prefill attention's vector instructions)
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]
# host code that uses the HIP runtime (streams, memory) and the kernel libraries' entry points
HIPHOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                 "-I/opt/rocm/include"]

# library name -> (compiler kind, sources relative to csrc, headers that also enter the hash)
LIBRARIES: Dict[str, dict] = {
    "runtime": {
        "kind": "cxx",
        "sources": ["runtime/cache_manager.cc", "runtime/scheduler.cc", "runtime/c_api.cc"],
        "headers": ["runtime/cache_manager.h", "runtime/scheduler.h"],
    },
    # plain C++ twins of the device operations: the oracle of the kernel tests (host only)
    "ref": {"kind": "cxx", "sources": ["ref/ref_ops.cc"], "headers": []},
    "elementwise": {"kind": "hip", "sources": ["kernels/elementwise.hip"], "headers": ["kernels/common.h"]},
    "gemm_f32": {"kind": "hip", "sources": ["kernels/gemm_f32.hip"], "headers": ["kernels/common.h"]},
    "gemm_bf16": {"kind": "hip", "sources": ["kernels/gemm_bf16.hip"], "headers": ["kernels/common.h"]},
    "attention": {"kind": "hip", "sources": ["kernels/attention.hip"], "headers": ["kernels/common.h"]},
    "attention_decode": {"kind": "hip", "sources": ["kernels/attention_decode.hip"], "headers": ["kernels/common.h"]},
    "attention_prefill": {"kind": "hip", "sources": ["kernels/attention_prefill.hip"], "headers": ["kernels/common.h"]},
    "sampling": {"kind": "hip", "sources": ["kernels/sampling.hip"],
                 "headers": ["kernels/common.h", "kernels/noalloc.h"]},
    "peaks": {"kind": "hip", "sources": ["kernels/peaks.hip"], "headers": ["kernels/common.h"]},
    # the native engine: checked dispatch over the kernels, the parts, the model's step function
    # (host code only; it calls the kernel libraries' entry points)
    "engine": {
        "kind": "hiphost",
        "sources": ["engine/ops.cc", "engine/parts.cc", "engine/json.cc", "engine/weights.cc", "engine/arch.cc",
                    "engine/gpt2.cc", "engine/engine.cc", "engine/engine_api.cc"],
        "headers": ["engine/ops.h", "engine/parts.h", "engine/kernels.h", "engine/json.h", "engine/weights.h",
                    "engine/arch.h", "engine/engine.h", "runtime/cache_manager.h", "runtime/scheduler.h"],
        "needs": ["elementwise", "gemm_f32", "gemm_bf16", "attention", "attention_decode", "attention_prefill",
                  "sampling", "runtime"],
    },
    # the command line: a program, not a library (mini_llm_amd/_lib/mini-llm; bin/mini-llm starts it)
    "cli": {
        "kind": "hiphost",
        "program": "mini-llm",
        "sources": ["engine/main.cc"],
        "headers": ["engine/engine.h", "engine/arch.h", "engine/weights.h", "engine/parts.h", "engine/ops.h",
                    "engine/json.h", "runtime/cache_manager.h", "runtime/scheduler.h"],
        "needs": ["engine", "runtime"],
    },
}



def register_library(name: str, spec: dict) -> None:
    """Adds a library to build: ``spec`` as in LIBRARIES, with absolute paths for ``sources`` and ``headers``
    and ``out_dir`` for the folder the built file goes to. ``kind: "plugin"`` is one hipcc source (host code
    that registers parts and architectures, and their kernels) linked against the engine library."""
    LIBRARIES[name] = spec


_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[mini_llm_amd build] {msg}", file=sys.stderr, flush=True)


def _paths(name: str):
    spec = LIBRARIES[name]
    srcs = [os.path.join(CSRC, s) for s in spec["sources"]]
    hdrs = [os.path.join(CSRC, h) for h in spec.get("headers", [])]
    return spec, srcs, hdrs


def _source_hash(name: str) -> str:
    spec, srcs, hdrs = _paths(name)
    h = hashlib.sha256()
    flags = {"hip": HIPCC_FLAGS, "cxx": CXX_FLAGS, "hiphost": HIPHOST_FLAGS, "plugin": HIPCC_FLAGS}[spec["kind"]]
    h.update(" ".join(flags).encode())
    if spec["kind"] == "plugin":
        # a plugin sees the engine's classes: it is stale when their headers change
        hdrs = hdrs + [os.path.join(CSRC, x) for x in LIBRARIES["engine"]["headers"]]
    for p in srcs + hdrs:
        with open(p, "rb") as f:
            h.update(os.path.relpath(p, CSRC).encode())
            h.update(f.read())
    return h.hexdigest()


def lib_path(name: str) -> str:
    program = LIBRARIES[name].get("program")
    return os.path.join(LIBRARIES[name].get("out_dir", LIB_DIR), program if program else f"libmllm_{name}.so")


def is_current(name: str) -> bool:
    so, stamp = lib_path(name), lib_path(name) + ".hash"
    if not (os.path.isfile(so) and os.path.isfile(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == _source_hash(name)


def needed_by(name: str) -> List[str]:
    """Every library that `name` links against, directly or through another."""
    out: List[str] = []
    for dep in LIBRARIES[name].get("needs", []):
        for d in needed_by(dep) + [dep]:
            if d not in out:
                out.append(d)
    return out


def _find(tool: str, extra: List[str]) -> str:
    p = shutil.which(tool)
    if p:
        return p
    for d in extra:
        c = os.path.join(d, tool)
        if os.path.isfile(c):
            return c
    raise BuildError(f"'{tool}' not found on PATH or in {extra}")


def build_library(name: str, verbose: bool = True) -> str:
    """Compiles one library unconditionally and returns its path."""
    spec, srcs, _ = _paths(name)
    out_dir = spec.get("out_dir", LIB_DIR)
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(out_dir, exist_ok=True)
    so = lib_path(name)
    link: List[str] = []
    if spec["kind"] == "hip":
        cc = _find("hipcc", ["/opt/rocm/bin"])
        cmd = [cc] + HIPCC_FLAGS
    elif spec["kind"] == "plugin":
        if not is_current("engine"):
            build_library("engine", verbose)
        cc = _find("hipcc", ["/opt/rocm/bin"])
        cmd = [cc] + HIPCC_FLAGS
        link = [f"-L{LIB_DIR}", "-lmllm_engine", f"-Wl,-rpath,{LIB_DIR}"]
    elif spec["kind"] == "hiphost":
        # link against the libraries beside it; stale ones are compiled first, those without needs of
        # their own side by side
        stale = [d for d in needed_by(name) if not is_current(d)]
        leaves = [d for d in stale if not LIBRARIES[d].get("needs")]
        if len(leaves) > 1:
            from concurrent.futures import ThreadPoolExecutor
            with ThreadPoolExecutor(max_workers=4) as ex:
                list(ex.map(lambda d: build_library(d, verbose), leaves))
        for dep in stale:
            if not is_current(dep):
                build_library(dep, verbose)
        cc = _find("g++", ["/usr/bin"])
        cmd = [cc] + [f for f in HIPHOST_FLAGS if not (spec.get("program") and f in ("-shared",))]
        link = [f"-L{LIB_DIR}"] + [f"-lmllm_{d}" for d in needed_by(name)] + \
               ["-L/opt/rocm/lib", "-lamdhip64", "-ldl", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    else:
        cc = _find("g++", ["/usr/bin"])
        cmd = [cc] + CXX_FLAGS
    # Compile to a private name, then rename: a concurrent process never sees a half-written file.
    fd, tmp = tempfile.mkstemp(prefix=f".{name}.", suffix=".tmp" if spec.get("program") else ".so", dir=out_dir)
    os.close(fd)
    cmd = cmd + [f"-I{os.path.join(CSRC, 'kernels')}", f"-I{os.path.join(CSRC, 'runtime')}",
                 f"-I{os.path.join(CSRC, 'engine')}"] + srcs + ["-o", tmp] + link
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    if verbose:
        _say(f"compiling {name} ({', '.join(spec['sources'])}) ...")
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    out_lines: List[str] = []

    def _drain():
        for line in proc.stdout:
            out_lines.append(line)

    th = threading.Thread(target=_drain, daemon=True)
    th.start()
    while proc.poll() is None:
        th.join(timeout=15)
        if proc.poll() is None and verbose:
            _say(f"  ... still compiling {name} ({time.time() - t0:.0f} s)")
    th.join()
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise BuildError(f"building {name} failed:\n{' '.join(cmd)}\n{''.join(out_lines)}")
    os.replace(tmp, so)
    os.chmod(so, 0o755)
    with open(so + ".hash", "w") as f:
        f.write(_source_hash(name))
    if verbose:
        _say(f"built {name} in {time.time() - t0:.1f} s")
    return so


def build_all(verbose: bool = True, jobs: int = 4) -> None:
    """Compiles every library, whatever is there already."""
    from concurrent.futures import ThreadPoolExecutor
    first = [n for n in LIBRARIES if not LIBRARIES[n].get("needs")]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda n: build_library(n, verbose), first))
    for n in LIBRARIES:                     # then those that link against others
        if n not in first:
            build_library(n, verbose)
    with _lock:
        _loaded.clear()


_runtime_shared = False


def _share_hip_runtime_with_torch() -> None:
    """One HIP runtime per process. PyTorch-ROCm bundles a copy of the HIP runtime and loads it by another
    file name than the system's, so a process that loads the system's copy first (through these libraries)
    and imports torch afterwards ends up with two runtimes, and the second finds no GPU. If torch is
    installed and not imported yet, its copy is therefore loaded first, by path, without importing torch:
    these libraries then bind to it (it carries the system copy's name), as they do when torch came first."""
    global _runtime_shared
    if _runtime_shared or "torch" in sys.modules:
        _runtime_shared = True
        return
    _runtime_shared = True
    try:
        import importlib.util
        spec = importlib.util.find_spec("torch")
        if spec is None or not spec.submodule_search_locations:
            return
        path = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
        if os.path.isfile(path):
            ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    except (OSError, ImportError, ValueError):
        pass          # no torch, or a torch without a bundled runtime: the system's copy is the only one


def load_library(name: str) -> ctypes.CDLL:
    """Loads a library, building it first if it is missing or out of date."""
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        if not is_current(name):
            build_library(name)
        if LIBRARIES[name]["kind"] != "cxx":
            _share_hip_runtime_with_torch()
        lib = ctypes.CDLL(lib_path(name))
        _loaded[name] = lib
        return lib
