"""Compiles the native code in-tree: the gfx950 kernels (hipcc) and the host runtime (g++).

These libraries are built into ``rust_llm_inference_server_amd/_lib``:

* ``librlis_kernels.so``   - ``kernels/*.hip`` but the matrix-core attention;
* ``librlis_attn_dN.so``   - the matrix-core attention (``kernels/attention_mfma.hip``) for head
  sizes up to N = 32, 64, ... 256, one library each: a model needs one of them, and only that
  one is built and loaded for it;
* ``librlis_runtime.so``   - ``runtime/*.cpp``: page manager and scheduler, no GPU needed.

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
# (no fused multiply-adds: the seeded weights must come out the same from any compiler)
CXX_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-Wall", "-pthread",
             "-ffp-contract=off"]

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


ATTENTION_UNIT_SOURCE = "attention_mfma.hip"


def attention_unit(head_dim: int) -> str:
    """The library kind that serves ``head_dim`` on the matrix cores."""
    padded = -(-head_dim // 32) * 32
    if padded not in MFMA_ATTENTION_HEAD_DIMS:
        raise ValueError(f"no matrix-core attention unit for head size {head_dim}")
    return f"attn_d{padded}"


def all_kinds() -> List[str]:
    return ["runtime", "kernels"] + [f"attn_d{d}" for d in MFMA_ATTENTION_HEAD_DIMS]


def _is_hip(kind: str) -> bool:
    return kind != "runtime"


def _sources(kind: str) -> List[str]:
    d = os.path.join(HERE, "kernels" if _is_hip(kind) else "runtime")
    if kind.startswith("attn_d"):
        return [os.path.join(d, ATTENTION_UNIT_SOURCE)]
    ext = (".hip",) if _is_hip(kind) else (".cpp",)
    return sorted(os.path.join(d, f) for f in os.listdir(d)
                  if f.endswith(ext) and f != ATTENTION_UNIT_SOURCE)


def _headers(kind: str) -> List[str]:
    d = os.path.join(HERE, "kernels" if _is_hip(kind) else "runtime")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith((".h", ".hpp")))


def _units(kind: str) -> List[Tuple[str, str, List[str]]]:
    """(object name, source, extra defines) for every compile step."""
    if kind.startswith("attn_d"):
        src, = _sources(kind)
        return [(f"attention_mfma_{kind[5:]}", src, [f"-DRLIS_HEAD_DIM={kind[6:]}"])]
    return [(os.path.splitext(os.path.basename(src))[0], src, []) for src in _sources(kind)]


def source_hash(kind: str) -> str:
    h = hashlib.sha256(kind.encode())
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


def build_many(kinds: Sequence[str], jobs: Optional[int] = None) -> List[str]:
    """Compile the libraries ``kinds`` from scratch (all their units through one pool) and
    return their paths."""
    lib_dir = _lib_dir()
    obj_dir = os.path.join(lib_dir, f"_build_{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    work: List[Tuple[str, Tuple[str, str, List[str]]]] = [(k, u) for k in kinds for u in _units(k)]
    jobs = jobs or min(8, os.cpu_count() or 1, len(work))
    _say(f"compiling {len(work)} units of {', '.join(kinds)} ({jobs} at a time)")

    def compile_one(item: Tuple[str, Tuple[str, str, List[str]]]) -> str:
        kind, (name, src, defs) = item
        cc, flags = (_hipcc(), HIP_FLAGS) if _is_hip(kind) else (shutil.which("g++") or "g++", CXX_FLAGS)
        obj = os.path.join(obj_dir, f"{kind}.{name}.o")
        _say(f"  {name} ...")
        _run([cc, *flags, *defs, "-c", src, "-o", obj], f"  {name}")
        return obj

    objs: Dict[str, List[str]] = {k: [] for k in kinds}
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for (kind, _), obj in zip(work, pool.map(compile_one, work)):
            objs[kind].append(obj)
    outs = []
    for kind in kinds:
        out = lib_path(kind)
        tmp = out + f".tmp{os.getpid()}"
        if _is_hip(kind):
            link = [_hipcc(), f"--offload-arch={ARCH}", "-fPIC", "-shared", "-o", tmp, *objs[kind]]
        else:
            link = [shutil.which("g++") or "g++", "-shared", "-pthread", "-o", tmp, *objs[kind]]
        _run(link, f"linking {os.path.basename(out)}")
        os.replace(tmp, out)
        with open(out + ".hash", "w") as f:
            f.write(source_hash(kind))
        outs.append(out)
    shutil.rmtree(obj_dir, ignore_errors=True)
    return outs


def build(kind: str, jobs: Optional[int] = None) -> str:
    """Compile library ``kind`` ('kernels', 'runtime' or an attention unit) from scratch."""
    return build_many([kind], jobs)[0]


def ensure(kind: str) -> str:
    """Path of library ``kind``; built first when absent or older than its sources."""
    if not is_current(kind):
        _say(f"librlis_{kind}.so is absent or out of date; building it now")
        build(kind)
    return lib_path(kind)


def build_all() -> None:
    build_many(all_kinds())


if __name__ == "__main__":
    build_all()
