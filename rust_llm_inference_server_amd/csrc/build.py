"""Compiles the native code in-tree: the gfx950 kernels (hipcc) and the host runtime (g++).

Two libraries are built into ``rust_llm_inference_server_amd/_lib``:

* ``librlis_kernels.so``  - every ``kernels/*.hip`` (and the per-head-size attention units);
* ``librlis_runtime.so``  - ``runtime/*.cpp``: page manager and scheduler, no GPU needed.

``ensure(name)`` returns the path of a library, building it first when it is absent or older
than its sources; a line is printed before each compile step so that a first call in a fresh
checkout shows progress.  When the package folder is not writable the libraries go to a
folder under the system's temporary directory instead.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import Dict, List, Optional, Sequence, Tuple

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    # Packed float32 forms are kept out of the generated code.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # Matrix-core results go to ordinary vector registers: the softmax and the epilogues read
    # them with vector instructions, and copies out of the accumulator file cost as much.
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wno-unused-command-line-argument",
]
CXX_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-Wall"]

# Head sizes (rounded up to a multiple of 32) the matrix-core attention unit is built for.
MFMA_ATTENTION_HEAD_DIMS = (32, 64, 96, 128, 160, 192, 224, 256)


def _say(msg: str) -> None:
    print(f"[rlis build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _lib_dir() -> str:
    d = os.path.join(PKG, "_lib")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"rlis_amd_lib_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _sources(kind: str) -> List[str]:
    sub = "kernels" if kind == "kernels" else "runtime"
    ext = (".hip",) if kind == "kernels" else (".cpp",)
    d = os.path.join(HERE, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(ext))


def _headers(kind: str) -> List[str]:
    sub = "kernels" if kind == "kernels" else "runtime"
    d = os.path.join(HERE, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith((".h", ".hpp")))


def _units(kind: str) -> List[Tuple[str, str, List[str]]]:
    """(object name, source, extra defines) for every compile step."""
    units = []
    for src in _sources(kind):
        base = os.path.splitext(os.path.basename(src))[0]
        if kind == "kernels" and base == "attention_mfma":
            for d in MFMA_ATTENTION_HEAD_DIMS:
                units.append((f"{base}_d{d}", src, [f"-DRLIS_HEAD_DIM={d}"]))
        else:
            units.append((base, src, []))
    return units


def source_hash(kind: str) -> str:
    h = hashlib.sha256()
    for path in _sources(kind) + _headers(kind) + [os.path.abspath(__file__)]:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def lib_path(kind: str) -> str:
    return os.path.join(_lib_dir(), f"librlis_{kind}.so")


def is_current(kind: str) -> bool:
    p = lib_path(kind)
    stamp = p + ".hash"
    if not (os.path.exists(p) and os.path.exists(stamp)):
        return False
    with open(stamp, "r") as f:
        return f.read().strip() == source_hash(kind)


def _run(cmd: Sequence[str], what: str) -> None:
    t0 = time.time()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{proc.stdout}")
    _say(f"{what} done in {time.time() - t0:.1f}s")


def build(kind: str, jobs: Optional[int] = None) -> str:
    """Compile library ``kind`` ('kernels' or 'runtime') from scratch and return its path."""
    out = lib_path(kind)
    obj_dir = os.path.join(os.path.dirname(out), f"_build_{kind}")
    os.makedirs(obj_dir, exist_ok=True)
    units = _units(kind)
    if kind == "kernels":
        cc, flags = _hipcc(), HIP_FLAGS
    else:
        cc, flags = shutil.which("g++") or "g++", CXX_FLAGS
    jobs = jobs or min(8, os.cpu_count() or 1, len(units))
    _say(f"compiling {len(units)} {kind} units with {os.path.basename(cc)} ({jobs} at a time)")
    objs: Dict[str, str] = {}

    def compile_one(unit: Tuple[str, str, List[str]]) -> str:
        name, src, defs = unit
        obj = os.path.join(obj_dir, name + ".o")
        _say(f"  {name} ...")
        _run([cc, *flags, *defs, "-c", src, "-o", obj], f"  {name}")
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for unit, obj in zip(units, pool.map(compile_one, units)):
            objs[unit[0]] = obj
    tmp = out + f".tmp{os.getpid()}"
    link = [cc, "-shared", "-o", tmp, *objs.values()]
    if kind == "kernels":
        link[1:1] = [f"--offload-arch={ARCH}", "-fPIC"]
    _run(link, f"linking {os.path.basename(out)}")
    os.replace(tmp, out)
    with open(out + ".hash", "w") as f:
        f.write(source_hash(kind))
    shutil.rmtree(obj_dir, ignore_errors=True)
    return out


def ensure(kind: str) -> str:
    """Path of library ``kind``; built first when absent or older than its sources."""
    if not is_current(kind):
        _say(f"librlis_{kind}.so is absent or out of date; building it now")
        build(kind)
    return lib_path(kind)


def build_all() -> None:
    build("runtime")
    build("kernels")


if __name__ == "__main__":
    build_all()
