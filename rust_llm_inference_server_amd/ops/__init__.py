"""The kernels as Python functions over torch tensors on the GPU.

Each function checks on the host that shapes, dtypes, strides and alignment are what its
kernel and grid assume, then launches on torch's current stream.  Nothing here computes on
the CPU; without the compiled library or without a GPU the first call raises.
"""
from __future__ import annotations

import ctypes
import functools
import math
import weakref
from typing import Optional, Tuple

import torch

from ..stepplan import StepPlan
from . import lib
from .attention_plan import AttentionPlanner
from .lib import KernelError

_DT = {torch.float32: 0, torch.bfloat16: 1}

# bf16 products with at most this many rows of x take the skinny kernel (where the library's
# GEMM is not used, see BF16_GEMM).
SKINNY_MAX_ROWS = 64
# ... and with at most this many rows the streaming kernel (16 at most; 0 switches it off).
STREAM_MAX_ROWS = 16
# ... and, where the rows are short enough for a wave to keep 32 of them in registers (k up to
# 3072), with up to this many rows its form for 17 to 32 rows (0 switches that off: such steps
# then take the library's products, the split-k kernel and the norm and SwiGLU kernels).
STREAM_WIDE_MAX_ROWS = 32
# A product whose result joins the residual stream as partial sums (``partials=True``) takes the
# split-k kernel from 17 rows up to this many (64 at most; 0 switches it off).
SPLITK_MAX_ROWS = 64
# Single tokens in a batch that also holds portions of prompts take the decode attention kernel.
SPLIT_MIXED_ATTENTION = True
# The norm in front of a projection goes into the streaming kernel where that applies.
FUSE_NORM_LINEAR = True
# A projection whose result joins the residual stream in front of such a norm adds it there
# itself and hands the norm's sums over, so that the product behind the norm needs no pass over
# whole rows (up to 16 rows, one k slice on both sides).
JOIN_NORM_LINEAR = True
# The matrix-core decode attention rotates q and k and stores the new k, v itself where it can.
FUSE_ROPE_DECODE = True
# The matrix-core prefill attention rotates its queries as it loads them where it can (the
# rotation kernel then turns and stores the keys and values only).
FUSE_ROPE_PREFILL = True
# "library": bf16 products with more rows than the streaming kernel takes go to torch
# (hipBLASLt); "own": they take the hand-written skinny and matrix-core kernels.
BF16_GEMM = "library"
# The library's products are called directly (hipBLASLt's own entry points, a plan kept per
# shape) rather than through torch.matmul: the same library and algorithm, two thirds of the
# host time per call.
LIBRARY_GEMM_DIRECT = True
# None: attention kernels are chosen from the batch; "generic": the generic kernel always
# (what the command line's --attention v1 asks for).
FORCE_ATTENTION: Optional[str] = None
# "matrix": bfloat16 decode attention on the matrix cores where it applies; "vector": always
# the vector-unit decode kernel (tests compare the two).
DECODE_ATTENTION = "matrix"
# The matrix-core decode attention merges a sequence's partitions in the workgroup that finishes
# last instead of in a second kernel (the same sums either way; tests compare the two).  The
# workgroups count themselves in in ``counters``, int32 zeros that the caller owns (a model's
# runner brings its own, so two runners on two streams do not count into each other's; a call
# without them gets a set that all such calls on the device share, one stream at a time).
# It pays while the kernel is short: every
# workgroup ends with a round trip to memory in which it streams nothing, about 3 % of a long
# kernel's time, against the 5 us of the second kernel; so it is used up to this many bytes of
# keys and values under the grid (partitions x partition length x 2 x head size x 2 bytes: an
# upper bound, since a captured step's grid is as deep as its context bucket's longest context
# needs and most sequences are shorter; 64 requests of the 3B shape with contexts up to 2,300,
# 1.07 GB by this count, gain 3 % of their step inside; 32 requests of the 8B shape at 8,300,
# 1.125 GB, take the same time either way).  Grids whose workgroups walk several partitions
# merge inside whatever their size: their workgroups are few.
MERGE_DECODE_INSIDE = True
MERGE_DECODE_INSIDE_MAX_BYTES = 9 << 27        # 1.125 GB
# The most partitions that one workgroup of that kernel takes in a row: None = by how many
# workgroups the batch makes (``attention_plan.decode_shares``), a number = that many, dealt
# out to as few workgroups as that allows (tests: the floats are the same however a sequence's
# partitions are dealt out).
DECODE_WALK: Optional[int] = None


_shared_counters: dict = {}


def _counters_for(device: torch.device) -> torch.Tensor:
    """The arrival counters of callers that bring none: one set per device, made at first use
    (not under stream capture: a captured step brings its runner's)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    c = _shared_counters.get(index)
    if c is None:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention: a captured step must bring its own counters")
        c = _shared_counters[index] = torch.zeros(1 << 16, dtype=torch.int32, device=device)
    return c


@functools.lru_cache(maxsize=None)
def _compute_units_of(index: int) -> int:
    return int(torch.cuda.get_device_properties(index).multi_processor_count)


def _compute_units(device: torch.device) -> int:
    return _compute_units_of(device.index if device.index is not None
                             else torch.cuda.current_device())


# A product over a long k whose result joins the residual stream (the consumer takes a stack of
# partial sums) at the row counts of a budgeted step: the library's kernels for one such
# product are few workgroups with long loops over k; as one batched call over slices of k they
# are more and shorter (3B shape, down projection at 512 rows: 51 -> 36 us, against which the
# consumer reads 25 MB more).  Rows and k from which on, rows up to which; eight slices up to
# LIBRARY_SLICES_FINE_ROWS rows and four beyond (with the norm behind it and the library's
# candidates tried out, k = 8,192 at 128 / 512 rows: one product 33 / 52 us, four slices 25 /
# 40, eight 24.5 / 43; k = 14,336: one 57 / 97, four 40 / 72, seven 48 / 90, eight 38 / 76,
# fourteen 46 / 99), two from LIBRARY_SLICES_MID_ROWS rows on (at 2,048 rows k = 8,192 of the
# 1B shape 88.6 -> 84.2 us, k = 14,336 239 -> 227; four slices lose there), fewer where k does
# not divide into slices whose rows stay 16-byte aligned.
LIBRARY_SLICES_MIN_ROWS = 65
LIBRARY_SLICES_MAX_ROWS = 2048
LIBRARY_SLICES_MIN_K = 8192
LIBRARY_SLICES_FINE_ROWS = 256
LIBRARY_SLICES_MID_ROWS = 1024


def library_slices(T: int, K: int) -> int:
    """k slices of the library's product at ``T`` rows over ``K`` when its consumer takes
    partial sums (1: one product).  It follows from the row count and k alone."""
    if not (LIBRARY_SLICES_MIN_ROWS <= T <= LIBRARY_SLICES_MAX_ROWS) or K < LIBRARY_SLICES_MIN_K:
        return 1
    counts = ((8, 4, 2) if T <= LIBRARY_SLICES_FINE_ROWS else
              (4, 2) if T <= LIBRARY_SLICES_MID_ROWS else (2,))
    for slices in counts:
        if K % (slices * 8) == 0:
            return slices
    return 1


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype} (float32 and bfloat16 only)") from None


def _check(t: torch.Tensor, name: str, dtype=None, ndim: Optional[int] = None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, kernels run on the GPU only")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise KernelError(f"{name}: expected {ndim} dimensions, got shape {tuple(t.shape)}")


def _rows_contig(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    _check(t, name, ndim=2)
    if t.shape[1] > 1 and t.stride(1) != 1:
        raise KernelError(f"{name}: rows must be contiguous, strides are {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> int:
    _check(t, name, torch.int32)
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name}: needs {n} entries, has {t.numel()}")
    return t.data_ptr()


# --------------------------------------------------------------------------- rows
def embed(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Rows ``table[ids]`` as the float32 residual stream ``(T, H)``."""
    _check(table, "embed table", ndim=2)
    T, (V, H) = ids.numel(), table.shape
    if not table.is_contiguous():
        raise KernelError("embed table must be contiguous")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    lib.call("rlis_embed", out.data_ptr(), table.data_ptr(), _dt(table), _i32(ids, "ids", T),
             T, H, lib.stream_ptr())
    return out


def _delta_parts(resid: torch.Tensor, delta: torch.Tensor, what: str) -> int:
    """A delta is shaped like the residual, or is a stack ``(S, T, H)`` of float32 partial sums
    (what ``linear(..., partials=True)`` returns) that are added in order."""
    _check(delta, "delta")
    if not delta.is_contiguous():
        raise KernelError(f"{what}: delta must be contiguous")
    if delta.shape == resid.shape:
        return 1
    if delta.dim() == resid.dim() + 1 and delta.shape[1:] == resid.shape \
            and delta.dtype == torch.float32 and delta.shape[0] >= 1:
        return delta.shape[0]
    raise KernelError(f"{what}: delta of shape {tuple(delta.shape)} does not match the residual "
                      f"{tuple(resid.shape)}")


def add_residual(resid: torch.Tensor, delta: torch.Tensor, round_parts: bool = False) -> None:
    """``resid += delta`` with the sum formed in float32.  ``round_parts``: a stack of partial
    sums (of one slice or of many) is added up and rounded to bfloat16 before it joins the
    residual."""
    _check(resid, "residual", torch.float32)
    if not resid.is_contiguous():
        raise KernelError("add_residual: residual must be contiguous")
    parts = _delta_parts(resid, delta, "add_residual")
    lib.call("rlis_add_residual", resid.data_ptr(), delta.data_ptr(), _dt(delta), resid.numel(),
             parts, int(bool(round_parts) and delta.dim() > resid.dim()), lib.stream_ptr())


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                write_resid: bool = True, round_parts: bool = False) -> torch.Tensor:
    """``norm(resid + delta) * weight`` row by row (``round_parts`` as in ``add_residual``).

    With ``rows`` only those rows are produced and the residual is left as it is; otherwise
    the sum is stored back into ``resid`` when ``write_resid`` is set."""
    _check(resid, "residual", torch.float32, 2)
    T, H = resid.shape
    if not resid.is_contiguous():
        raise KernelError("add_rmsnorm: residual must be contiguous")
    parts = 1 if delta is None else _delta_parts(resid, delta, "add_rmsnorm")
    _check(weight, "norm weight", ndim=1)
    if weight.numel() != H or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: weight has {weight.numel()} entries, rows have {H}")
    if rows is not None:
        R, rows_ptr, write_resid = rows.numel(), _i32(rows, "rows"), False
    else:
        R, rows_ptr = T, None
    out = torch.empty((R, H), dtype=out_dtype, device=resid.device)
    lib.call("rlis_add_rmsnorm", resid.data_ptr(),
             None if delta is None else delta.data_ptr(), 0 if delta is None else _dt(delta),
             weight.data_ptr(), _dt(weight), out.data_ptr(), _DT[out_dtype], rows_ptr, R, H,
             float(eps), int(bool(write_resid)), parts, T * H,
             int(bool(round_parts) and delta is not None and delta.dim() > resid.dim()),
             lib.stream_ptr())
    return out


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    """``silu(gu[:, :I]) * gu[:, I:]`` for ``gu`` of shape ``(T, 2 I)``."""
    _check(gu, "gate/up", ndim=2)
    T, two_i = gu.shape
    if two_i % 2 or not gu.is_contiguous():
        raise KernelError("swiglu: input must be contiguous with an even number of columns")
    out = torch.empty((T, two_i // 2), dtype=gu.dtype, device=gu.device)
    lib.call("rlis_swiglu", out.data_ptr(), gu.data_ptr(), _dt(gu), T, two_i // 2,
             lib.stream_ptr())
    return out


# ----------------------------------------------------------------------- products
def stream_slices(K: int) -> int:
    """Number of k slices the streaming kernel cuts a plain product over ``K`` into."""
    return lib.load().rlis_gemm_bf16_stream_slices(K)


def stream_rows(K: int) -> int:
    """The most rows of ``x`` that the streaming kernels take for rows of ``K``."""
    if STREAM_MAX_ROWS < 16 or STREAM_WIDE_MAX_ROWS <= 16:
        return STREAM_MAX_ROWS
    return max(16, min(STREAM_WIDE_MAX_ROWS, lib.load().rlis_gemm_bf16_stream_max_rows(K)))


def _one_item_per_wave(K: int) -> bool:
    """Whether a row of ``K`` fits the streaming kernel's forms that take one k item per wave
    (the fused norm, the gated and the scaled form)."""
    return K <= lib.load().rlis_norm_linear_max_k()


# The library's products of 33 to 1,024 rows are tried out before a shape's first product: the
# heuristics' first candidates are timed on the spot and the fastest is kept for the shape
# (``rlis_lt_tune``; their order is erratic at these sizes, see library_gemm.hip), over the
# weights of up to sixteen layers in turn, so that no candidate finds its weights in a cache
# (timed on four weights of 31 MB, which the memory-side cache holds, the pick for the 3B
# shape's q/k/v at 640 rows was 7 % slower in a step than the heuristics' first).  A
# shape is tried out once, before anything has used it, and keeps its algorithm from then on: a
# step computes the same bits whenever it runs.  Row counts beyond 64 are tried out when they
# are a multiple of 32 (what a token budget makes of most steps) or named in
# ``LIBRARY_TUNE_ROWS`` (an engine names its token budget); the others take the algorithm of
# the next multiple of 32 (``rlis_lt_adopt``: the candidate of their own that names the same
# kernel, untimed), and under a capturing stream every new shape takes the heuristics' first.
LIBRARY_TUNE = True
LIBRARY_TUNE_MAX_ROWS = 1024
LIBRARY_TUNE_CANDIDATES = 12
LIBRARY_TUNE_MARGIN = 0.08       # the first candidate stays unless another is this much faster
LIBRARY_TUNE_ROWS: set = set()   # further row counts to try out (an engine's token budget)
LIBRARY_TUNE_BYTES = 512 << 20   # weights that the timed products of a candidate walk over
_tried_out: set = set()
_same_shape: dict = {}           # (device index, N, K, row stride) -> {address: weak reference}
tune_log: list = []              # (T, N, K, slices, candidate taken, us of the first, us of it)
adopt_log: list = []             # (T, rows it follows, N, K, slices, candidate taken or -1)


def note_weights(tensors) -> None:
    """Tells the tuner which weights a model holds: products are tried out over the weights of
    one shape in turn (two-dimensional bfloat16 tensors; anything else is skipped)."""
    for t in tensors:
        if (isinstance(t, torch.Tensor) and t.dim() == 2 and t.dtype == torch.bfloat16
                and t.is_cuda and t.stride(1) == 1):
            key = (t.device.index, t.shape[0], t.shape[1], t.stride(0))
            _same_shape.setdefault(key, {})[t.data_ptr()] = weakref.ref(t)


def _try_out(x, w, y, out_f32, T, N, K, ldx, ldw, slices, ws, stream, partial=False) -> None:
    if not LIBRARY_TUNE or T > (LIBRARY_SLICES_MAX_ROWS if slices > 1 else LIBRARY_TUNE_MAX_ROWS):
        return                  # (in slices of k the heuristics' first is not the best at 2,048 rows either)
    key = (x.device.index, T, N, K, ldx, ldw, bool(out_f32), slices)
    if key in _tried_out:
        return
    _tried_out.add(key)
    if torch.cuda.is_current_stream_capturing():
        return
    if T > 64 and T % 32 and T not in LIBRARY_TUNE_ROWS:
        # A row count between two that are tried out takes the algorithm of the next one up
        # (tried out now, on rows of nothing, when it has not been yet): the same kernel does
        # as well for a few rows fewer, and nothing more is timed.
        like = -(-T // 32) * 32
        like_slices = library_slices(like, K) if partial else 1
        if like > (LIBRARY_SLICES_MAX_ROWS if slices > 1 else LIBRARY_TUNE_MAX_ROWS) or like_slices != slices:
            return
        if (x.device.index, like, N, K, K, ldw, bool(out_f32), slices) not in _tried_out:
            rows = torch.empty((like, K), dtype=torch.bfloat16, device=x.device)
            out = torch.empty((slices, like, N) if partial and slices > 1 else (like, N),
                              dtype=y.dtype, device=x.device)
            _try_out(rows, w, out, out_f32, like, N, K, K, ldw, slices, ws, stream, partial)
        taken = ctypes.c_int(-1)
        lib.call("rlis_lt_adopt", T, like, int(out_f32), N, K, ldx, K, ldw, N, slices, T * N,
                 ws.numel(), ctypes.byref(taken))
        adopt_log.append((T, like, N, K, slices, taken.value))
        return
    # as many weights as make up LIBRARY_TUNE_BYTES (the memory-side cache is 256 MB), 4 to 16
    most = max(4, min(16, -(-LIBRARY_TUNE_BYTES // (N * K * 2))))
    held = [w]                                        # (strong references while they are used)
    for ref in list(_same_shape.get((x.device.index, N, K, ldw), {}).values()):
        t = ref()
        if t is not None and t.data_ptr() != w.data_ptr() and len(held) < most:
            held.append(t)
    ptrs = (ctypes.c_void_p * len(held))(*[t.data_ptr() for t in held])
    chosen = ctypes.c_int(-1)
    us = (ctypes.c_float * 2)()
    lib.call("rlis_lt_tune", x.data_ptr(), ptrs, len(held), y.data_ptr(), int(out_f32), T, N, K,
             ldx, ldw, N, slices, T * N, ws.data_ptr(), ws.numel(), LIBRARY_TUNE_CANDIDATES,
             2 if len(held) < 8 else 1, LIBRARY_TUNE_MARGIN, ctypes.byref(chosen), us, stream)
    if chosen.value >= 0:
        tune_log.append((T, N, K, slices, chosen.value, float(us[0]), float(us[1])))


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           partials: bool = False) -> torch.Tensor:
    """``x @ w.T`` for ``x (T, K)`` and ``w (N, K)``, float32 accumulation.

    A float32 weight (or float32 ``x``) takes the plain FMA kernel, the true 32-bit product.
    bfloat16 operands take the streaming kernel up to 16 rows; more rows go to the library's
    GEMM (hipBLASLt, through its own entry points), or with ``BF16_GEMM = "own"`` to the skinny
    kernel up to 64 rows and the hand-written matrix-core GEMM beyond.

    ``partials``: the caller hands the result to the residual stream and takes it as a stack
    ``(S, T, N)`` of float32 partial sums too (one per k slice of the streaming kernel, or of
    the split-k kernel that 17 to 64 rows take, added in order by ``add_rmsnorm`` /
    ``add_residual``) where that saves a pass."""
    ldx = _rows_contig(x, "linear x")
    ldw = _rows_contig(w, "linear weight")
    T, K = x.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"linear: x has {K} columns, the weight {K2}")
    out_dtype = out_dtype or x.dtype
    stream = lib.stream_ptr()
    bf16 = x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    aligned = (K % 8 == 0 and ldx % 8 == 0 and ldw % 8 == 0
               and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
    if bf16 and aligned and STREAM_MAX_ROWS < T <= stream_rows(K):
        # 17 to 32 rows over a k that a wave holds in registers: one result, whoever asks
        y = torch.empty((T, N), dtype=out_dtype, device=x.device)
        lib.call("rlis_gemm_bf16_stream", x.data_ptr(), w.data_ptr(), y.data_ptr(),
                 _DT[y.dtype], T, N, K, ldx, ldw, N, T * N, 0, stream)
        return y
    if bf16 and aligned and partials and STREAM_MAX_ROWS < T <= SPLITK_MAX_ROWS:
        slices = lib.load().rlis_gemm_bf16_splitk_slices(N, K)
        y = torch.empty((slices, T, N), dtype=torch.float32, device=x.device)
        lib.call("rlis_gemm_bf16_splitk", x.data_ptr(), w.data_ptr(), y.data_ptr(), T, N, K, ldx,
                 ldw, T * N, stream)
        return y
    if bf16 and aligned and T > STREAM_MAX_ROWS and BF16_GEMM == "library":
        ws = lib.library_workspace(x.device) if LIBRARY_GEMM_DIRECT else None
        slices = library_slices(T, K) if partials and ws is not None else 1
        if slices > 1:
            y = torch.empty((slices, T, N), dtype=torch.float32, device=x.device)
            _try_out(x, w, y, True, T, N, K, ldx, ldw, slices, ws, stream, partial=True)
            lib.call("rlis_lt_gemm_bf16_slices", x.data_ptr(), w.data_ptr(), y.data_ptr(), T, N, K,
                     ldx, ldw, N, slices, T * N, ws.data_ptr(), ws.numel(), stream)
            return y
        if ws is not None and out_dtype in (torch.bfloat16, torch.float32):
            y = torch.empty((T, N), dtype=out_dtype, device=x.device)
            _try_out(x, w, y, out_dtype == torch.float32, T, N, K, ldx, ldw, 1, ws, stream)
            lib.call("rlis_lt_gemm_bf16", x.data_ptr(), w.data_ptr(), y.data_ptr(),
                     int(out_dtype == torch.float32), T, N, K, ldx, ldw, N, ws.data_ptr(),
                     ws.numel(), stream)
            return y
        if out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t())
        return torch.mm(x, w.t(), out_dtype=torch.float32)    # float32 accumulation and result
    if bf16 and aligned and 0 < T <= STREAM_MAX_ROWS:
        slices = stream_slices(K)
        if slices == 1 or partials:
            if slices == 1:
                y = torch.empty((T, N), dtype=out_dtype, device=x.device)
            else:
                y = torch.empty((slices, T, N), dtype=torch.float32, device=x.device)
            lib.call("rlis_gemm_bf16_stream", x.data_ptr(), w.data_ptr(), y.data_ptr(),
                     _DT[y.dtype], T, N, K, ldx, ldw, N, T * N, 0, stream)
            return y
    y = torch.empty((T, N), dtype=out_dtype, device=x.device)
    if T == 0:
        return y
    if bf16 and aligned:
        name = "rlis_gemm_bf16_skinny" if T <= SKINNY_MAX_ROWS else "rlis_gemm_bf16_mfma"
        lib.call(name, x.data_ptr(), w.data_ptr(), y.data_ptr(), _DT[out_dtype], T, N, K, ldx,
                 ldw, N, stream)
    else:
        lib.call("rlis_gemm_plain", x.data_ptr(), _dt(x), w.data_ptr(), _dt(w), y.data_ptr(),
                 _DT[out_dtype], T, N, K, ldx, ldw, N, stream)
    return y


def can_fuse_norm_linear(resid: torch.Tensor, w: torch.Tensor, rows: Optional[int] = None
                         ) -> bool:
    """Whether ``norm_linear`` applies: at most 16 rows, a bfloat16 weight over one k slice."""
    T = resid.shape[0] if rows is None else rows
    K = resid.shape[1]
    return (0 < T <= STREAM_MAX_ROWS and FUSE_NORM_LINEAR and w.dtype == torch.bfloat16
            and w.dim() == 2 and w.shape[1] == K and K % 8 == 0 and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
            and K <= lib.load().rlis_norm_linear_max_k())


def norm_linear(resid: torch.Tensor, delta: Optional[torch.Tensor], norm_weight: torch.Tensor,
                eps: float, w: torch.Tensor, out_dtype: torch.dtype, gated: bool = False,
                rows: Optional[torch.Tensor] = None, round_parts: bool = False):
    """RMSNorm of ``resid + delta`` and the product with ``w`` in one kernel (see
    ``can_fuse_norm_linear``); ``gated`` as ``linear_swiglu``, ``round_parts`` as in
    ``add_residual``.  Returns ``(y, resid_sum)``:
    without ``rows``, ``resid_sum`` is ``resid + delta`` in a new tensor (``resid`` itself when
    there is no delta); with ``rows``, only those rows are produced and ``resid_sum`` is None."""
    _check(resid, "residual", torch.float32, 2)
    T, K = resid.shape
    if not resid.is_contiguous():
        raise KernelError("norm_linear: residual must be contiguous")
    parts = 1 if delta is None else _delta_parts(resid, delta, "norm_linear")
    _check(norm_weight, "norm weight", ndim=1)
    if norm_weight.numel() != K or not norm_weight.is_contiguous():
        raise KernelError(f"norm_linear: norm weight has {norm_weight.numel()} entries, rows {K}")
    ldw = _rows_contig(w, "norm_linear weight")
    if w.shape[1] != K or w.dtype != torch.bfloat16:
        raise KernelError("norm_linear: the weight must be bfloat16 (N, K)")
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("norm_linear: a gated weight needs an even number of rows")
        N //= 2
    if rows is not None:
        R, rows_ptr, resid_sum = rows.numel(), _i32(rows, "rows"), None
    else:
        R, rows_ptr = T, None
        resid_sum = resid if delta is None else torch.empty_like(resid)
    y = torch.empty((R, N), dtype=out_dtype, device=resid.device)
    if R:
        lib.call("rlis_norm_linear_bf16", resid.data_ptr(),
                 None if delta is None else delta.data_ptr(), 0 if delta is None else _dt(delta),
                 parts, T * K,
                 int(bool(round_parts) and delta is not None and delta.dim() > resid.dim()),
                 norm_weight.data_ptr(),
                 _dt(norm_weight), float(eps), rows_ptr,
                 None if (delta is None or rows is not None) else resid_sum.data_ptr(),
                 w.data_ptr(), y.data_ptr(), _DT[out_dtype], R, N, K, ldw, N, int(bool(gated)),
                 lib.stream_ptr())
    return y, resid_sum


class PendingProduct:
    """``x @ w.T`` on its way into the residual stream, not run yet: the norm that follows can
    then run it with the residual add and its own multiplies inside (``linear_join_norm``);
    ``run()`` is the plain product, as ``linear(..., partials=True)`` gives it."""

    __slots__ = ("x", "w", "out_dtype")

    def __init__(self, x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype]):
        self.x, self.w, self.out_dtype = x, w, out_dtype

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.x.shape[0], self.w.shape[0])

    def run(self) -> torch.Tensor:
        return linear(self.x, self.w, self.out_dtype, partials=True)


def _streams_in_one_slice(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dim() == 2 and w.dim() == 2 and x.dtype == torch.bfloat16
            and w.dtype == torch.bfloat16 and 0 < x.shape[0] <= stream_rows(x.shape[1])
            and x.shape[1] == w.shape[1] and x.shape[1] % 8 == 0 and stream_slices(x.shape[1]) == 1
            and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def pending_linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None):
    """The projection whose result joins the residual stream: ``linear(x, w, out_dtype,
    partials=True)``, or where the norm behind it may take it in (``JOIN_NORM_LINEAR``; up to 16
    rows of bfloat16, one k slice, an output width that the next product can read as its rows)
    a ``PendingProduct`` that has not run."""
    if JOIN_NORM_LINEAR and _streams_in_one_slice(x, w) and w.shape[0] % 8 == 0:
        return PendingProduct(x, w, out_dtype)
    return linear(x, w, out_dtype, partials=True)


def can_join_norm_linear(product: PendingProduct, resid: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``linear_join_norm`` and ``linear_scaled`` take this product, residual and the
    weight of the product behind the norm."""
    T, H = resid.shape
    return (JOIN_NORM_LINEAR and resid.dtype == torch.float32 and resid.is_contiguous()
            and product.shape == (T, H) and w.dim() == 2 and w.shape[1] == H
            and w.dtype == torch.bfloat16 and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0 and _one_item_per_wave(H) and T <= stream_rows(H)
            # (17 to 32 rows: the scaled form takes up to 256 partial sums of squares a row)
            and (T <= 16 or lib.load().rlis_gemm_bf16_stream_join_tiles(H, product.x.shape[1]) <= 256))


def linear_join_norm(product: PendingProduct, resid: torch.Tensor, norm_weight: torch.Tensor,
                     round_sum: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Runs the product with what follows it inside: ``resid += x @ w.T`` (the product rounded
    to bfloat16 first with ``round_sum``, as a bfloat16 model's block output is), in place.
    Returns ``(xw, ss)``: ``resid * norm_weight`` in bfloat16 and, ``(16, tiles)`` float32, per
    row and tile of columns the sum of ``resid ** 2`` (rows from ``T`` on are not meant), for
    ``linear_scaled``."""
    x, w = product.x, product.w
    T, K = x.shape
    N = w.shape[0]
    _check(norm_weight, "norm weight", ndim=1)
    if norm_weight.numel() != N or not norm_weight.is_contiguous():
        raise KernelError(f"linear_join_norm: norm weight has {norm_weight.numel()} entries, "
                          f"rows have {N}")
    tiles = lib.load().rlis_gemm_bf16_stream_join_tiles(N, K)
    if tiles <= 0:
        raise KernelError("linear_join_norm: cannot read the device properties")
    xw = torch.empty((T, N), dtype=torch.bfloat16, device=x.device)
    stride = -(-tiles // 4) * 4
    ss = torch.empty((-(-T // 16) * 16, stride), dtype=torch.float32, device=x.device)[:, :tiles]
    lib.call("rlis_gemm_bf16_stream_join", x.data_ptr(), w.data_ptr(), T, N, K, x.stride(0),
             w.stride(0), resid.data_ptr(), resid.data_ptr(), norm_weight.data_ptr(),
             _dt(norm_weight), int(bool(round_sum)), xw.data_ptr(), ss.data_ptr(), stride,
             lib.stream_ptr())
    return xw, ss


def linear_scaled(xw: torch.Tensor, ss: torch.Tensor, eps: float, w: torch.Tensor,
                  out_dtype: torch.dtype, gated: bool = False) -> torch.Tensor:
    """``(xw * rsqrt(mean of the rows' squares + eps)) @ w.T`` (``gated`` as ``linear_swiglu``),
    the rows' sums of squares given as ``linear_join_norm`` leaves them: the RMSNorm of the
    residual and the product behind it."""
    T, K = xw.shape
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("linear_scaled: a gated weight needs an even number of rows")
        N //= 2
    y = torch.empty((T, N), dtype=out_dtype, device=xw.device)
    lib.call("rlis_gemm_bf16_stream_scaled", xw.data_ptr(), w.data_ptr(), y.data_ptr(),
             _DT[out_dtype], T, N, K, xw.stride(0), w.stride(0), N, int(bool(gated)),
             ss.data_ptr(), ss.shape[1], ss.stride(0), float(eps), lib.stream_ptr())
    return y


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]`` of shape ``(2 I, K)``.

    Up to 16 rows of bfloat16 (64 with ``BF16_GEMM = "own"``) take one kernel that never stores
    the ``(T, 2 I)`` intermediate; everything else is the product followed by the SwiGLU
    kernel."""
    T, K = x.shape
    two_i = w_gate_up.shape[0]
    if two_i % 2:
        raise KernelError("linear_swiglu: the fused weight needs an even number of rows")
    ldx = _rows_contig(x, "linear_swiglu x")
    ldw = _rows_contig(w_gate_up, "linear_swiglu weight")
    fusable = (x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
               and 0 < T and K == w_gate_up.shape[1] and K % 8 == 0
               and ldx % 8 == 0 and ldw % 8 == 0 and x.data_ptr() % 16 == 0
               and w_gate_up.data_ptr() % 16 == 0)
    streamed = fusable and T <= stream_rows(K) and _one_item_per_wave(K)
    skinny = fusable and not streamed and T <= SKINNY_MAX_ROWS and \
        (BF16_GEMM == "own" or T <= STREAM_MAX_ROWS)
    if not (streamed or skinny):
        return swiglu(linear(x, w_gate_up, x.dtype))
    y = torch.empty((T, two_i // 2), dtype=torch.bfloat16, device=x.device)
    if streamed:
        lib.call("rlis_gemm_bf16_stream", x.data_ptr(), w_gate_up.data_ptr(), y.data_ptr(), 1, T,
                 two_i // 2, K, ldx, ldw, two_i // 2, 0, 1, lib.stream_ptr())
    else:
        lib.call("rlis_gemm_bf16_skinny_swiglu", x.data_ptr(), w_gate_up.data_ptr(), y.data_ptr(),
                 T, two_i // 2, K, ldx, ldw, two_i // 2, lib.stream_ptr())
    return y


# ------------------------------------------------------------ rotation + cache write
def rope_kv_write(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                  cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  positions: torch.Tensor, slots: Optional[torch.Tensor],
                  k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
                  page_size: int, write_kv: bool = True, interleaved: bool = False,
                  rotate_q: bool = True) -> None:
    """Rotate the q and k heads of ``qkv (T, (nh + 2 nkv) d)`` by their positions (q in
    place; not at all without ``rotate_q``, for a consumer that turns q as it loads it) and,
    when ``write_kv``, store rotated k and v into the pages at ``slots``.
    The rotation pairs dim ``j`` with ``j + rot/2`` (rotate-half, the reference's), or with
    ``interleaved`` dim ``2j`` with ``2j + 1``.

    ``cos``/``sin`` are float32 ``(max_positions, rot_dim / 2)``; None means no rotation.
    ``k_pages (pages, nkv, page, d)``, ``v_pages (pages, nkv, d, page)``."""
    stride = _rows_contig(qkv, "qkv")
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    if qkv.shape[1] != (nh + 2 * nkv) * d:
        raise KernelError(f"rope_kv_write: qkv has {qkv.shape[1]} columns, expected "
                          f"{(nh + 2 * nkv) * d}")
    if cos is None:
        rot, cos_ptr, sin_ptr = 0, None, None
    else:
        _check(cos, "cos", torch.float32, 2)
        _check(sin, "sin", torch.float32, 2)
        if cos.shape != sin.shape or not (cos.is_contiguous() and sin.is_contiguous()):
            raise KernelError("rope_kv_write: cos and sin must match and be contiguous")
        rot, cos_ptr, sin_ptr = 2 * cos.shape[1], cos.data_ptr(), sin.data_ptr()
        if rot > d:
            raise KernelError(f"rope_kv_write: rotation width {rot} exceeds head_dim {d}")
    kp = vp = sp = None
    if write_kv:
        if k_pages is None or v_pages is None or slots is None:
            raise KernelError("rope_kv_write: a cache write needs pages and slots")
        for t, name, shape in ((k_pages, "k_pages", (nkv, page_size, d)),
                               (v_pages, "v_pages", (nkv, d, page_size))):
            _check(t, name, qkv.dtype, 4)
            if tuple(t.shape[1:]) != shape or not t.is_contiguous():
                raise KernelError(f"rope_kv_write: {name} has shape {tuple(t.shape)}, expected "
                                  f"(pages, {shape[0]}, {shape[1]}, {shape[2]}) contiguous")
        kp, vp, sp = k_pages.data_ptr(), v_pages.data_ptr(), _i32(slots, "slots", T)
    lib.call("rlis_rope_kv_write", qkv.data_ptr(), _dt(qkv), stride, nh * d, (nh + nkv) * d, T,
             nh, nkv, d, rot, cos_ptr, sin_ptr, _i32(positions, "positions", T), sp, kp, vp,
             page_size, int(bool(write_kv)), int(bool(interleaved)), int(bool(rotate_q)),
             lib.stream_ptr())


def copy_pages(pages: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """``pages (layers, num_pages, ...)``: copy page ``src[i]`` onto ``dst[i]`` in every layer."""
    _check(pages, "pages")
    if pages.dim() < 3 or not pages.is_contiguous():
        raise KernelError("copy_pages: pages must be (layers, num_pages, ...) contiguous")
    n = src.numel()
    if dst.numel() != n:
        raise KernelError("copy_pages: src and dst differ in length")
    page_elems = pages[0, 0].numel()
    lib.call("rlis_copy_pages", pages.data_ptr(), _dt(pages), pages.shape[0], pages.shape[1],
             page_elems, _i32(src, "src"), _i32(dst, "dst"), n, lib.stream_ptr())


# ----------------------------------------------------------------------- attention
def _decode_mfma_ok(qkv: torch.Tensor, nh: int, nkv: int, d: int, page_size: int) -> bool:
    """Whether single tokens of this layout can take the matrix-core decode kernel."""
    g = nh // nkv
    return (qkv.dtype == torch.bfloat16 and d % 16 == 0 and d <= 256 and g <= 16
            and g * (d + 2) * 32 <= 65536 and AttentionPlanner.pages_fit(page_size)
            and qkv.stride(0) % 8 == 0 and DECODE_ATTENTION != "vector")


def _prefill_mfma_ok(qkv: torch.Tensor, d: int, page_size: int) -> bool:
    return (qkv.dtype == torch.bfloat16 and d % 16 == 0 and d <= 256
            and AttentionPlanner.pages_fit(page_size) and qkv.stride(0) % 8 == 0)


def attention_planner(num_heads: int, num_kv_heads: int, head_dim: int,
                      dtype: torch.dtype, biased: bool = False) -> AttentionPlanner:
    """The planner a mixer that calls ``paged_attention`` / ``rope_attention`` names as its
    ``step_planner()``; ``biased``: it will pass ``bias_slopes`` (the matrix-core kernels take
    them too, so the plan is the same)."""
    return AttentionPlanner(num_heads, num_kv_heads, head_dim,
                            matrix=dtype == torch.bfloat16,
                            singles_apart=SPLIT_MIXED_ATTENTION and DECODE_ATTENTION != "vector")


def _attention_kernel(qkv: torch.Tensor, nh: int, nkv: int, d: int, page_size: int, step,
                      force: Optional[str], biased: bool = False):
    """(kind, matrix_decode): which attention kernel a batch takes.  A bias on the scores
    changes nothing here: every kernel takes one."""
    kind = force or FORCE_ATTENTION
    if kind is None:
        if step.all_decode and d % 8 == 0 and d <= 256 and (nh // nkv) * d <= 2048:
            kind = "decode"
        elif _prefill_mfma_ok(qkv, d, page_size) and not step.all_decode:
            kind = "prefill"
        else:
            kind = "generic"
    mfma = kind == "decode" and _decode_mfma_ok(qkv, nh, nkv, d, page_size)
    return kind, mfma


def _plan_now(step, planner: AttentionPlanner, device: torch.device) -> StepPlan:
    """A plan made on the spot from the step's host lengths (callers outside a model: tests,
    probes); a model's steps bring theirs, made by the step builder."""
    lengths = getattr(step, "lengths", None)
    if lengths is None:
        raise KernelError("attention: the step brings neither a plan nor its host lengths")
    host = planner.plan(lengths)
    arrays = {k: torch.from_numpy(v).to(device) for k, v in host.arrays.items()}
    return StepPlan(arrays, host.values)


def rope_attention(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                   positions: torch.Tensor, slots: Optional[torch.Tensor],
                   k_pages: torch.Tensor, v_pages: torch.Tensor, page_size: int,
                   block_tables: torch.Tensor, step, scale: float,
                   window: Optional[int] = None, write_kv: bool = True,
                   plan: Optional[StepPlan] = None, interleaved: bool = False,
                   bias_slopes: Optional[torch.Tensor] = None,
                   counters: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``rope_kv_write`` followed by ``paged_attention``.  A decode batch that takes the
    matrix-core decode kernel does both in that kernel when the whole head is rotated
    (rotate-half) and is 64, 128 or 256 wide (or nothing is rotated); ``qkv`` is then left
    unrotated.  Under the same conditions a batch with portions of prompts leaves the queries
    unrotated too: ``rope_kv_write`` turns and stores the keys and values alone, and the
    matrix-core kernels (prefill for the portions, decode for single tokens beside them) turn
    each query as they load it.  ``interleaved`` and ``bias_slopes`` as in ``rope_kv_write``
    and ``paged_attention``."""
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    _rows_contig(qkv, "qkv")
    kind, mfma = _attention_kernel(qkv, nh, nkv, d, page_size, step, None, bias_slopes is not None)
    fusable = cos is None or (2 * cos.shape[1] == d and d in (64, 128, 256) and not interleaved)
    whole_rows = qkv.shape[1] == (nh + 2 * nkv) * d
    if cos is not None and fusable and whole_rows and (mfma or kind == "prefill"):
        _check(cos, "cos", torch.float32, 2)
        _check(sin, "sin", torch.float32, 2)
        if cos.shape != sin.shape or not (cos.is_contiguous() and sin.is_contiguous()):
            raise KernelError("rope_attention: cos and sin must match and be contiguous")
    if mfma and fusable and FUSE_ROPE_DECODE and whole_rows:
        if write_kv and slots is None:
            raise KernelError("rope_attention: a cache write needs slots")
        return paged_attention(qkv, nh, nkv, d, k_pages, v_pages, page_size, block_tables, step,
                               scale, window, plan=plan, counters=counters,
                               bias_slopes=bias_slopes,
                               rope=(cos, sin, positions, slots if write_kv else None))
    if (kind == "prefill" and cos is not None and fusable and FUSE_ROPE_PREFILL and whole_rows
            and (_decode_mfma_ok(qkv, nh, nkv, d, page_size)
                 or (plan is not None and not plan.value("num_decode")))):
        rope_kv_write(qkv, nh, nkv, d, cos, sin, positions, slots, k_pages, v_pages, page_size,
                      write_kv=write_kv, rotate_q=False)
        return paged_attention(qkv, nh, nkv, d, k_pages, v_pages, page_size, block_tables, step,
                               scale, window, plan=plan, counters=counters,
                               bias_slopes=bias_slopes, rope=(cos, sin, positions, None))
    rope_kv_write(qkv, nh, nkv, d, cos, sin, positions, slots, k_pages, v_pages, page_size,
                  write_kv=write_kv, interleaved=interleaved)
    return paged_attention(qkv, nh, nkv, d, k_pages, v_pages, page_size, block_tables, step,
                           scale, window, plan=plan, bias_slopes=bias_slopes, counters=counters)


def paged_attention(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                    k_pages: torch.Tensor, v_pages: torch.Tensor, page_size: int,
                    block_tables: torch.Tensor, step, scale: float,
                    window: Optional[int] = None, force: Optional[str] = None,
                    rope: Optional[tuple] = None, plan: Optional[StepPlan] = None,
                    bias_slopes: Optional[torch.Tensor] = None,
                    counters: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the step's new tokens over the paged cache -> ``(T, nh * d)``.

    ``qkv`` holds the rotated queries in its first ``nh * d`` columns; K and V of the new
    tokens are already in the pages.  ``step`` is the ``StepContext`` (token and sequence
    metadata on the device), ``plan`` what an ``AttentionPlanner`` made for it (made on the
    spot from ``step.lengths`` when absent).  The kernel is chosen from the shape of the
    batch: every sequence brings one token -> decode kernel; bfloat16 with multi-token
    sequences -> matrix-core prefill kernel (single tokens that lead the step beside them ->
    decode kernel); float32, or sizes those kernels refuse -> generic kernel.  How a sequence's
    keys are cut (decode partitions, tile form, key runs) follows from its own lengths alone.
    ``bias_slopes`` (float32, one per query head; the reference has no such thing): the score of
    key position ``u`` for a query at position ``p`` gets ``slope * (u - p)`` added before the
    softmax; every kernel takes it (the matrix-core ones in a form of their own).
    ``force`` names one of 'generic', 'decode', 'prefill' for tests.  ``rope`` (from
    ``rope_attention`` only): ``(cos, sin, positions, slots)`` for the matrix-core decode kernel
    to rotate and store the step's tokens itself; with portions of prompts in the batch
    ``slots`` is None (the pages hold the step's keys and values already) and both matrix-core
    kernels turn the unrotated queries as they load them.  ``counters``: int32 zeros on the device, the
    caller's, in which the matrix-core decode kernel's workgroups count themselves in when they
    merge partitions inside the kernel (they leave zeros); launches that may overlap in time
    must not share them."""
    q_stride = _rows_contig(qkv, "qkv")
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    if nh % nkv:
        raise KernelError(f"attention: {nh} query heads are not a multiple of {nkv} KV heads")
    for t, name, shape in ((k_pages, "k_pages", (nkv, page_size, d)),
                           (v_pages, "v_pages", (nkv, d, page_size))):
        _check(t, name, qkv.dtype, 4)
        if tuple(t.shape[1:]) != shape or not t.is_contiguous():
            raise KernelError(f"attention: {name} has shape {tuple(t.shape)}, expected "
                              f"(pages, {shape[0]}, {shape[1]}, {shape[2]}) contiguous")
    _check(block_tables, "block_tables", torch.int32, 2)
    if block_tables.shape[0] < step.num_seqs or not block_tables.is_contiguous():
        raise KernelError("attention: block table rows do not cover the step's sequences")
    max_pages = block_tables.shape[1]
    need_pages = -(-step.max_context // page_size)
    if max_pages < need_pages:
        raise KernelError(f"attention: block tables hold {max_pages} pages per sequence, the "
                          f"longest context needs {need_pages}")
    if T != step.num_tokens:
        raise KernelError(f"attention: qkv has {T} rows, the step {step.num_tokens} tokens")
    win = int(window) if window else 0
    out = torch.empty((T, nh * d), dtype=qkv.dtype, device=qkv.device)
    stream = lib.stream_ptr()
    slopes_ptr = None
    if bias_slopes is not None:
        _check(bias_slopes, "bias_slopes", torch.float32, 1)
        if bias_slopes.numel() != nh or not bias_slopes.is_contiguous():
            raise KernelError(f"attention: {bias_slopes.numel()} bias slopes for {nh} heads")
        slopes_ptr = bias_slopes.data_ptr()
    kind, mfma = _attention_kernel(qkv, nh, nkv, d, page_size, step, force, slopes_ptr is not None)
    if rope is not None and not (mfma or (kind == "prefill" and rope[3] is None
                                          and rope[0] is not None)):
        raise KernelError("attention: only the matrix-core kernels rotate, and only the decode "
                          "kernel stores")
    if kind == "generic":
        lib.call("rlis_attn_generic", qkv.data_ptr(), _dt(qkv), q_stride, out.data_ptr(), nh * d,
                 k_pages.data_ptr(), v_pages.data_ptr(), block_tables.data_ptr(), max_pages,
                 _i32(step.seq_of_token, "seq_of_token", T), _i32(step.positions, "positions", T),
                 T, nh, nkv, d, page_size, float(scale), win, slopes_ptr, stream)
        return out
    if kind not in ("decode", "prefill"):
        raise KernelError(f"attention: unknown kernel '{kind}'")
    if plan is None or force == "prefill":
        planner = AttentionPlanner(nh, nkv, d, matrix=qkv.dtype == torch.bfloat16,
                                   singles_apart=force is None and SPLIT_MIXED_ATTENTION
                                   and DECODE_ATTENTION != "vector")
        plan = _plan_now(step, planner, qkv.device)

    def decode(S: int, depth: int, matrix: bool) -> None:
        """The first S sequences, one token each (their token rows are the first S too)."""
        from . import attention_plan as ap
        part_ml = part_acc = None
        if depth > 1:
            part_ml = torch.empty((S, nh, depth, 2), dtype=torch.float32, device=qkv.device)
            part_acc = torch.empty((S, nh, depth, d), dtype=torch.float32, device=qkv.device)
        ml_ptr = None if part_ml is None else part_ml.data_ptr()
        acc_ptr = None if part_acc is None else part_acc.data_ptr()
        if matrix:
            lib.ensure_attention_unit(d)
            cos_p = sin_p = pos_p = slots_p = None
            rot = 0
            if rope is not None:
                cos, sin, positions, slots = rope
                pos_p = _i32(positions, "positions", S)
                slots_p = None if slots is None else _i32(slots, "slots", S)
                if cos is not None:
                    cos_p, sin_p, rot = cos.data_ptr(), sin.data_ptr(), 2 * cos.shape[1]
            if DECODE_WALK:
                groups, cap = -(-depth // DECODE_WALK), DECODE_WALK
            else:
                groups, cap = ap.decode_shares(S, nkv, depth, nh // nkv, d,
                                               _compute_units(qkv.device))
            # (workgroups that take several partitions are few, and hand over little or nothing)
            inside = depth > 1 and MERGE_DECODE_INSIDE and (
                cap > 1 or S * nkv * depth * ap.DECODE_PART_KEYS * d * 4
                <= MERGE_DECODE_INSIDE_MAX_BYTES)
            arrivals_p, arrival_slots = None, 0
            if inside:
                arrivals = counters if counters is not None else _counters_for(qkv.device)
                arrivals_p, arrival_slots = _i32(arrivals, "counters", 1), arrivals.numel()
            lib.call("rlis_attn_decode_mfma", qkv.data_ptr(), q_stride, out.data_ptr(), nh * d,
                     ml_ptr, acc_ptr, k_pages.data_ptr(), v_pages.data_ptr(),
                     block_tables.data_ptr(), max_pages, _i32(step.ctx_lens, "ctx_lens", S), S,
                     nh, nkv, d, page_size, win, float(scale), depth, ap.DECODE_PART_KEYS,
                     ap.DECODE_MAX_PARTS, arrivals_p, arrival_slots, groups, cap, cos_p, sin_p,
                     rot, pos_p, slots_p, nh * d, (nh + nkv) * d, slopes_ptr, stream)
        else:
            lib.call("rlis_attn_decode", qkv.data_ptr(), _dt(qkv), q_stride, out.data_ptr(),
                     nh * d, ml_ptr, acc_ptr, k_pages.data_ptr(), v_pages.data_ptr(),
                     block_tables.data_ptr(), max_pages, _i32(step.ctx_lens, "ctx_lens", S), None,
                     S, nh, nkv, d, page_size, float(scale), win, depth, ap.DECODE_PART_KEYS,
                     ap.DECODE_MAX_PARTS, slopes_ptr, stream)

    if kind == "decode":
        if not step.all_decode:
            raise KernelError("attention: the decode kernel needs one token per sequence")
        if plan.value("num_decode") != step.num_seqs:
            raise KernelError("attention: the plan is not one of a step of single tokens")
        decode(step.num_seqs, plan.value("decode_depth"), mfma)
        return out
    if qkv.dtype != torch.bfloat16:
        raise KernelError("attention: the matrix-core prefill kernel is bfloat16 only")
    if not _prefill_mfma_ok(qkv, d, page_size):
        raise KernelError(f"attention: the matrix-core prefill kernel takes head sizes in steps "
                          f"of 16 up to 256 and pages of a power of two from 8 on, not head size "
                          f"{d} with pages of {page_size}")
    # Single tokens beside portions of prompts: the step lists them first, and the decode
    # kernel reads their keys and values once for the whole group of heads, where a tile of the
    # prefill kernel would walk the context for one query per head.
    singles = plan.value("num_decode")
    if singles:
        if not _decode_mfma_ok(qkv, nh, nkv, d, page_size):
            raise KernelError("attention: the plan sends single tokens to the matrix-core "
                              "decode kernel, which does not take this layout")
        decode(singles, plan.value("decode_depth"), True)
    row0, max_runs = plan.value("tile_row0"), plan.value("max_runs")
    part_ml = part_acc = None
    if max_runs > 1:
        part_ml = torch.empty((T - row0, nh, max_runs, 2), dtype=torch.float32, device=qkv.device)
        part_acc = torch.empty((T - row0, nh, max_runs, d), dtype=torch.float32, device=qkv.device)
    ml_ptr = None if part_ml is None else part_ml.data_ptr()
    acc_ptr = None if part_acc is None else part_acc.data_ptr()
    launched = False
    cos_p = sin_p = None
    rot = 0
    if rope is not None:
        cos_p, sin_p, rot = rope[0].data_ptr(), rope[1].data_ptr(), 2 * rope[0].shape[1]
    # Tiles of 64 queries, and tiles of 128 (two query blocks per wave, half the LDS traffic per
    # flop) for the sequences whose own lengths ask for them.
    for tile, name in ((64, "units64"), (128, "units128")):
        n = plan.value("num_" + name)
        if not n:
            continue
        lib.ensure_attention_unit(d)
        launched = True
        lib.call("rlis_attn_prefill_mfma", qkv.data_ptr(), q_stride, out.data_ptr(), nh * d,
                 k_pages.data_ptr(), v_pages.data_ptr(), block_tables.data_ptr(), max_pages,
                 _i32(step.cu_seqlens, "cu_seqlens", step.num_seqs + 1),
                 _i32(step.start_pos, "start_pos", step.num_seqs),
                 _i32(plan[name], name, 4 * n), n, nh, nkv, d, page_size, win, float(scale), tile,
                 max_runs, row0, ml_ptr, acc_ptr, cos_p, sin_p, rot, slopes_ptr, stream)
    if not launched and T > row0:
        raise KernelError("attention: the plan holds no tiles for the step's portions")
    if launched and max_runs > 1:
        # the runs of a sequence's tiles, merged as the decode kernel's partitions are
        lib.call("rlis_attn_reduce_rows", out.data_ptr(), nh * d, ml_ptr, acc_ptr,
                 _i32(step.seq_of_token, "seq_of_token", T),
                 _i32(plan["seq_runs"], "seq_runs", step.num_seqs), row0, T - row0, nh, d,
                 max_runs, stream)
    return out


# ------------------------------------------------------------------------ sampling
def sample_rows(logits: torch.Tensor, keys: torch.Tensor, inv_temps: torch.Tensor,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of float32 ``logits (R, V)``: argmax where ``inv_temps`` is 0, else
    Gumbel-max with noise keyed by ``keys`` (int32 bit patterns of the 32-bit row keys).  The
    tokens go to ``out`` (int32, ``R`` elements) when it is given."""
    stride = _rows_contig(logits, "logits")
    _check(logits, "logits", torch.float32)
    R, V = logits.shape
    _check(inv_temps, "inv_temps", torch.float32)
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    else:
        _i32(out, "sampled tokens", R)
    # A large vocabulary is scanned in chunks by many workgroups and a second small kernel
    # picks among the chunks' winners; the result is the same token.
    chunks = min(64, max(1, V // 1024))
    best = idx = None
    if chunks > 1:
        best = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        idx = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
    lib.call("rlis_sample_rows", logits.data_ptr(), stride, R, V, _i32(keys, "keys", R),
             inv_temps.data_ptr(), out.data_ptr(), chunks,
             None if best is None else best.data_ptr(), None if idx is None else idx.data_ptr(),
             lib.stream_ptr())
    return out


def fill_normal(out: torch.Tensor, seed: int, tensor_index: int, mean: float, std: float) -> None:
    """Fill ``out`` (float32 or bfloat16, contiguous, on the GPU) with ``mean + std * N(0, 1)``
    keyed by (seed, tensor index, element index): the generator of ``weights/random_init.py``,
    run on the device."""
    _check(out, "fill_normal out")
    if not out.is_contiguous():
        raise KernelError("fill_normal: the tensor must be contiguous")
    mask = (1 << 64) - 1
    lib.call("rlis_fill_normal_device", out.data_ptr(), _dt(out), out.numel(), int(seed) & mask,
             int(tensor_index) & mask, float(mean), float(std), lib.stream_ptr())


__all__ = ["AttentionPlanner", "KernelError", "add_residual", "add_rmsnorm", "attention_planner",
           "copy_pages", "embed", "fill_normal", "linear", "linear_swiglu", "norm_linear", "paged_attention",
           "rope_attention", "rope_kv_write", "sample_rows", "swiglu"]
