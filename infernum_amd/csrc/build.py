"""Builds the HIP sources of this folder for gfx950 with hipcc, into shared libraries.

There is one library for the kernels that every model needs, and one small
library per head size for the MFMA attention kernels, so that a first call
compiles what the model at hand needs and nothing else.  Libraries live in
``infernum_amd/_lib`` (or, where that folder cannot be written, under the
system's temporary folder).  ``ensure`` compiles a library only when it is not
there or its sources have changed; ``build_all`` always compiles.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import json
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List, Optional, Sequence

CSRC_DIR = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.dirname(CSRC_DIR)
ARCH = "gfx950"

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed fp32 instructions are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

CORE_SOURCES = [
    "elementwise.hip",
    "gemm_generic.hip",
    "gemm_skinny.hip",
    "gemm_mfma.hip",
    "attention_generic.hip",
    "sampling.hip",
    "peaks.hip",
]
HEADERS = ["common.h", "no_alloc.h", "op_call.h"]
# The host library: plain C++ (cache bookkeeping, packing of a step), built with the C++ compiler.
HOST_SOURCES = ["host_core.cpp", "step_program.cpp"]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]
# The binding of the vendor's GEMM library (hipBLASLt): host code too, against ROCm's headers and libraries.
BLASLT_SOURCES = ["gemm_library.cpp"]

# Head sizes whose attention library `build_all` compiles ahead of time.
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256)
SUPPORTED_HEAD_DIMS = tuple(range(16, 257, 16))


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[infernum_amd build] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def rocm_root() -> str:
    """Where ROCm's include/ and lib/ are: $ROCM_PATH, beside hipcc, or /opt/rocm."""
    cands = [os.environ.get("ROCM_PATH")]
    hipcc = find_hipcc()
    if hipcc:
        cands.append(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))))
    cands.append("/opt/rocm")
    for c in cands:
        if c and os.path.isfile(os.path.join(c, "include", "hipblaslt", "hipblaslt.h")):
            return c
    return "/opt/rocm"


def find_cxx() -> Optional[str]:
    """A C++ compiler for the host library; hipcc (a clang) serves when there is no other."""
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 find_hipcc()):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


_lib_dir: Optional[str] = None
_lib_dir_lock = threading.Lock()


def lib_dir() -> str:
    """Folder for built libraries: in the package if writable, else a temporary one."""
    global _lib_dir
    with _lib_dir_lock:
        if _lib_dir is None:
            d = os.path.join(PKG_DIR, "_lib")
            try:
                os.makedirs(d, exist_ok=True)
                fd, probe = tempfile.mkstemp(prefix=".w", dir=d)
                os.close(fd)
                os.unlink(probe)
            except OSError:
                d = os.path.join(tempfile.gettempdir(), f"infernum_amd_lib_{os.getuid()}")
                os.makedirs(d, exist_ok=True)
            _lib_dir = d
        return _lib_dir


def _existing(files: Sequence[str]) -> List[str]:
    return [f for f in files if os.path.isfile(os.path.join(CSRC_DIR, f))]


def _fingerprint(sources: Sequence[str], defines: Sequence[str], host: bool = False) -> str:
    h = hashlib.sha256()
    for f in list(sources) + _existing(HEADERS):
        with open(os.path.join(CSRC_DIR, f), "rb") as fh:
            h.update(f.encode())
            h.update(fh.read())
    h.update(" ".join((CXX_FLAGS if host else HIPCC_FLAGS) + list(defines)).encode())
    return h.hexdigest()


def library_plan(name: str) -> Dict:
    """Sources and defines of a library by its name ('core', 'attn_d<D>', 'host' or 'blaslt')."""
    if name == "host":
        return {"sources": _existing(HOST_SOURCES), "defines": [], "host": True}
    if name == "blaslt":
        root = rocm_root()
        return {"sources": _existing(BLASLT_SOURCES), "host": True,
                "defines": ["-D__HIP_PLATFORM_AMD__", f"-I{os.path.join(root, 'include')}"],
                "link": [f"-L{os.path.join(root, 'lib')}", "-lhipblaslt", "-lamdhip64",
                         f"-Wl,-rpath,{os.path.join(root, 'lib')}"]}
    if name == "core":
        return {"sources": _existing(CORE_SOURCES), "defines": []}
    if name.startswith("attn_d"):
        d = int(name[len("attn_d"):])
        if d not in SUPPORTED_HEAD_DIMS:
            raise BuildError(f"no MFMA attention kernel for head size {d}: supported are multiples of 16 up to 256")
        # accumulators of the matrix cores in ordinary vector registers: the softmax rescales them with
        # vector instructions, which cannot reach the accumulation registers
        return {"sources": ["attention_mfma.hip"],
                "defines": [f"-DIA_HEAD_DIM={d}", "-mllvm", "-amdgpu-mfma-vgpr-form"]}
    raise BuildError(f"unknown library {name!r}")


def library_path(name: str) -> str:
    return os.path.join(lib_dir(), f"libinfernum_{name}.so")


def _stamp_path(name: str) -> str:
    return os.path.join(lib_dir(), f"libinfernum_{name}.json")


def _heartbeat(stop: threading.Event, what: str) -> None:
    t0 = time.time()
    while not stop.wait(15.0):
        _say(f"still compiling {what} ({time.time() - t0:.0f} s)")


def _compile_host_library(name: str, plan: Dict) -> str:
    cxx = find_cxx()
    if cxx is None:
        raise BuildError("no C++ compiler found for the host library (looked at $CXX, g++, c++, clang++, hipcc)")
    out = library_path(name)
    tmp_dir = tempfile.mkdtemp(prefix=f"ia_{name}_", dir=lib_dir())
    t0 = time.time()
    try:
        tmp_out = os.path.join(tmp_dir, "lib.so")
        cmd = [cxx] + CXX_FLAGS + list(plan["defines"]) + ["-shared", "-o", tmp_out] + \
            [os.path.join(CSRC_DIR, f) for f in plan["sources"]] + list(plan.get("link", []))
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, cwd=tmp_dir)
        if r.returncode != 0:
            raise BuildError(f"{os.path.basename(cxx)} failed on {', '.join(plan['sources'])}:\n{r.stderr[-6000:]}")
        os.replace(tmp_out, out)
        with open(_stamp_path(name), "w") as f:
            json.dump({"fingerprint": _fingerprint(plan["sources"], list(plan["defines"]) + list(plan.get("link", [])),
                                                   host=True)}, f)
    finally:
        shutil.rmtree(tmp_dir, ignore_errors=True)
    _say(f"built {os.path.basename(out)} in {time.time() - t0:.1f} s")
    return out


def compile_library(name: str) -> str:
    """Compile one library now, whether or not it is there already."""
    if library_plan(name).get("host"):
        return _compile_host_library(name, library_plan(name))
    hipcc = find_hipcc()
    if hipcc is None:
        raise BuildError("hipcc not found: the HIP kernels cannot be compiled (looked at $HIPCC, PATH, /opt/rocm/bin)")
    plan = library_plan(name)
    out = library_path(name)
    tmp_dir = tempfile.mkdtemp(prefix=f"ia_{name}_", dir=lib_dir())
    _say(f"compiling {name} for {ARCH}: {', '.join(plan['sources'])}")
    stop = threading.Event()
    hb = threading.Thread(target=_heartbeat, args=(stop, name), daemon=True)
    hb.start()
    t0 = time.time()
    try:
        def one(src: str) -> str:
            obj = os.path.join(tmp_dir, os.path.splitext(src)[0] + ".o")
            cmd = [hipcc] + HIPCC_FLAGS + plan["defines"] + ["-c", os.path.join(CSRC_DIR, src), "-o", obj]
            r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, cwd=tmp_dir)
            if r.returncode != 0:
                raise BuildError(f"hipcc failed on {src}:\n{r.stderr[-6000:]}")
            return obj

        workers = max(1, min(len(plan["sources"]), int(os.environ.get("MAX_JOBS", "8")), 16))
        with concurrent.futures.ThreadPoolExecutor(workers) as ex:
            objs = list(ex.map(one, plan["sources"]))
        tmp_out = os.path.join(tmp_dir, "lib.so")
        r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp_out] + objs,
                           stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, cwd=tmp_dir)
        if r.returncode != 0:
            raise BuildError(f"hipcc failed to link {name}:\n{r.stderr[-6000:]}")
        os.replace(tmp_out, out)
        with open(_stamp_path(name), "w") as f:
            json.dump({"fingerprint": _fingerprint(plan["sources"], plan["defines"])}, f)
    finally:
        stop.set()
        shutil.rmtree(tmp_dir, ignore_errors=True)
    _say(f"built {os.path.basename(out)} in {time.time() - t0:.1f} s")
    return out


def ensure(name: str) -> str:
    """Path of a library, compiled first if it is missing or older than its sources."""
    out = library_path(name)
    plan = library_plan(name)
    if os.path.isfile(out):
        try:
            with open(_stamp_path(name)) as f:
                if json.load(f).get("fingerprint") == _fingerprint(
                        plan["sources"], list(plan["defines"]) + list(plan.get("link", [])), host=bool(plan.get("host"))):
                    return out
        except (OSError, ValueError):
            pass
        if (find_cxx() if plan.get("host") else find_hipcc()) is None:
            _say(f"{os.path.basename(out)} may be older than its sources and no compiler is here: using it as is")
            return out
    return compile_library(name)


def build_all(head_dims: Sequence[int] = DEFAULT_HEAD_DIMS) -> List[str]:
    """Compile every library (the core one, and attention for the given head sizes)."""
    names = ["host", "blaslt", "core"]
    if os.path.isfile(os.path.join(CSRC_DIR, "attention_mfma.hip")):
        names += [f"attn_d{d}" for d in head_dims]
    workers = max(1, min(4, int(os.environ.get("MAX_JOBS", "8"))))
    with concurrent.futures.ThreadPoolExecutor(workers) as ex:
        return list(ex.map(compile_library, names))


if __name__ == "__main__":
    build_all()
