"""Loads the compiled kernel library and declares its C entry points.

There is no fallback: without a GPU, or without the library, every op raises.  The library
is built on first use when it is absent (``csrc/build.py``)."""
from __future__ import annotations

import contextlib
import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p
from typing import Optional

import torch

_LIB: Optional[ctypes.CDLL] = None

P, I, L, F = c_void_p, c_int, c_longlong, c_float

_SIGNATURES = {
    "rlis_embed": [P, P, I, P, I, I, P],
    "rlis_add_residual": [P, P, I, L, I, I, P],
    "rlis_add_rmsnorm": [P, P, I, P, I, P, I, P, I, I, F, I, I, L, I, P],
    "rlis_swiglu": [P, P, I, I, I, P],
    "rlis_rope_kv_write": [P, I, L, I, I, I, I, I, I, I, P, P, P, P, P, P, I, I, I, I, P],
    "rlis_copy_pages": [P, I, I, L, L, P, P, I, P],
    "rlis_gemm_plain": [P, I, P, I, P, I, I, I, I, L, L, L, P],
    "rlis_gemm_bf16_mfma": [P, P, P, I, I, I, I, L, L, L, P],
    "rlis_gemm_bf16_skinny": [P, P, P, I, I, I, I, L, L, L, P],
    "rlis_gemm_bf16_skinny_swiglu": [P, P, P, I, I, I, L, L, L, P],
    "rlis_gemm_bf16_stream": [P, P, P, I, I, I, I, L, L, L, L, I, P],
    "rlis_gemm_bf16_splitk": [P, P, P, I, I, I, L, L, L, P],
    "rlis_gemm_bf16_stream_join": [P, P, I, I, I, L, L, P, P, P, I, I, P, P, I, P],
    "rlis_gemm_bf16_stream_scaled": [P, P, P, I, I, I, I, L, L, L, I, P, I, I, F, P],
    "rlis_norm_linear_bf16": [P, P, I, I, L, I, P, I, F, P, P, P, P, I, I, I, I, L, L, I, P],
    "rlis_attn_generic": [P, I, L, P, L, P, P, P, I, P, P, I, I, I, I, I, F, I, P, P],
    "rlis_attn_decode": [P, I, L, P, L, P, P, P, P, P, I, P, P, I, I, I, I, I, F, I, I, I, I, P, P],
    "rlis_attn_decode_mfma": [P, L, P, L, P, P, P, P, P, I, P, I, I, I, I, I, I, F, I, I, I, P, I, I, I,
                              P, P, I, P, P, L, L, P, P],
    "rlis_attn_prefill_mfma": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, I, I, P, P,
                               P, P, I, P, P],
    "rlis_attn_reduce_rows": [P, L, P, P, P, P, I, I, I, I, I, P],
    "rlis_sample_rows": [P, L, I, I, P, P, P, I, P, P, P],
    "rlis_fill_normal_device": [P, I, L, ctypes.c_ulonglong, ctypes.c_ulonglong, ctypes.c_double,
                                ctypes.c_double, P],
    "rlis_lt_open": [c_char_p],
    "rlis_lt_gemm_bf16": [P, P, P, I, I, I, I, L, L, L, P, ctypes.c_size_t, P],
    "rlis_lt_gemm_bf16_slices": [P, P, P, I, I, I, L, L, L, I, L, P, ctypes.c_size_t, P],
}


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or a launch failed."""


def load() -> ctypes.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    if not torch.cuda.is_available():
        raise RuntimeError(
            "rust_llm_inference_server_amd needs an AMD GPU (gfx950): torch.cuda.is_available() "
            "is False and there is no CPU fallback"
        )
    from ..csrc import build
    path = build.ensure("kernels")
    lib = ctypes.CDLL(path)
    lib.rlis_last_error.restype = c_char_p
    lib.rlis_last_error.argtypes = []
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise RuntimeError(f"{path} does not export {name}; rebuild the kernels")
        fn.restype = c_int
        fn.argtypes = argtypes
    lib.rlis_gemm_bf16_stream_slices.restype = c_int
    lib.rlis_gemm_bf16_stream_slices.argtypes = [I]
    lib.rlis_gemm_bf16_splitk_slices.restype = c_int
    lib.rlis_gemm_bf16_splitk_slices.argtypes = [I, I]
    lib.rlis_gemm_bf16_stream_join_tiles.restype = c_int
    lib.rlis_gemm_bf16_stream_join_tiles.argtypes = [I, I]
    lib.rlis_attn_register_unit.restype = c_int
    lib.rlis_attn_register_unit.argtypes = [I, P, P]
    lib.rlis_norm_linear_max_k.restype = c_int
    lib.rlis_norm_linear_max_k.argtypes = []
    lib.rlis_lt_tune.restype = c_int
    lib.rlis_lt_tune.argtypes = [P, P, I, P, I, I, I, I, L, L, L, I, L, P, ctypes.c_size_t, I, I, F,
                                 P, P, P]
    lib.rlis_lt_adopt.restype = c_int
    lib.rlis_lt_adopt.argtypes = [I, I, I, I, I, L, L, L, L, I, L, ctypes.c_size_t, P]
    lib.rlis_gemm_bf16_stream_max_rows.restype = c_int
    lib.rlis_gemm_bf16_stream_max_rows.argtypes = [I]
    _LIB = lib
    library_workspace(torch.device("cuda", torch.cuda.current_device()))
    return lib


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


# ---------------------------------------------------------------- the library's products
# Workspace that hipBLASLt may use for a product (what the tensor library grants it on this
# family of chips): one per device and stream, since products on two streams may run at the
# same time (two runners on two threads, each on a stream of its own).  Allocated at the first
# product on a stream, never while a stream is capturing: a capture runs on a stream of its own
# for a graph that its owner replays on the owner's stream, so whoever captures names that
# stream (``workspace_owner``), and the graph's products take its workspace.
LT_WORKSPACE_BYTES = 76 << 20
_LT_OPEN: Optional[bool] = None
_LT_WORKSPACES: dict = {}          # (device index, stream handle) -> uint8 tensor
_LT_OWNER = threading.local()


def _hipblaslt_path() -> str:
    """The copy of hipBLASLt that this process has loaded already: the tensor library's own."""
    import os
    own = os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so")
    return own if os.path.exists(own) else "libhipblaslt.so"


@contextlib.contextmanager
def workspace_owner(stream: "torch.cuda.Stream"):
    """Inside the block, this thread's library products take the workspace of ``stream``
    whichever stream is current (the warm-up and the capture of a graph that will be replayed
    on ``stream``).  The workspace is made on entry, before anything captures."""
    old = getattr(_LT_OWNER, "stream", None)
    _LT_OWNER.stream = int(stream.cuda_stream)
    try:
        library_workspace(stream.device)
        yield
    finally:
        _LT_OWNER.stream = old


def library_workspace(device: torch.device) -> Optional[torch.Tensor]:
    """The workspace of the device's current stream (or of the stream that ``workspace_owner``
    names) for ``rlis_lt_gemm_bf16``, or None when the library's products cannot be called
    directly (its entry points were not found, or the workspace would have to be allocated
    under a capturing stream): the caller then goes through ``torch.matmul``, which reaches the
    same library."""
    global _LT_OPEN
    if _LT_OPEN is None:
        _LT_OPEN = load().rlis_lt_open(_hipblaslt_path().encode()) == 0
    if not _LT_OPEN:
        return None
    index = device.index if device.index is not None else torch.cuda.current_device()
    owner = getattr(_LT_OWNER, "stream", None)
    if owner is None:
        owner = (_RAW_STREAM(index) if _RAW_STREAM is not None
                 else torch.cuda.current_stream(index).cuda_stream)
    ws = _LT_WORKSPACES.get((index, owner))
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            return None
        ws = torch.empty(LT_WORKSPACE_BYTES, dtype=torch.uint8, device=torch.device("cuda", index))
        _LT_WORKSPACES[(index, owner)] = ws
    return ws


_UNITS: dict = {}      # padded head size -> the loaded unit library


def ensure_attention_unit(head_dim: int) -> None:
    """Build (when absent), load and register the matrix-core attention unit that serves
    ``head_dim``: a model needs one, and only that one is compiled for it."""
    padded = -(-head_dim // 32) * 32
    if padded in _UNITS:
        return
    main = load()
    from ..csrc import build
    try:
        kind = build.attention_unit(head_dim)
    except ValueError as e:
        raise KernelError(str(e)) from None
    unit = ctypes.CDLL(build.ensure(kind))
    fns = []
    for name in (f"rlis_attn_prefill_mfma_d{padded}", f"rlis_attn_decode_mfma_d{padded}"):
        fn = getattr(unit, name, None)
        if fn is None:
            raise RuntimeError(f"{unit._name} does not export {name}; rebuild the kernels")
        fns.append(ctypes.cast(fn, c_void_p))
    if main.rlis_attn_register_unit(padded, *fns) != 0:
        raise KernelError(main.rlis_last_error().decode("utf-8", "replace"))
    _UNITS[padded] = unit


def loaded_path() -> Optional[str]:
    return None if _LIB is None else _LIB._name


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.rlis_last_error().decode("utf-8", "replace"))


def stream_ptr() -> int:
    """torch's current HIP stream of the current device, as the kernels' launch argument."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(torch.cuda.current_device())    # the same stream, looked up faster
    return torch.cuda.current_stream().cuda_stream
