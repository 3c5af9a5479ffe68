"""The sampling entry point that allocates nothing (``rlis_sample_rows_static``), called through
``ctypes`` as a caller without torch would, against the existing ``rlis_sample_rows``: two calls
in a row on the same GPU, the second with a smaller input, so that what the first call left in
the static scratch must not show in the second."""
import ctypes
from ctypes import c_int, c_longlong, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _library():
    from rust_llm_inference_server_amd.csrc import build
    lib = ctypes.CDLL(build.ensure("kernels"))
    P, I, L = c_void_p, c_int, c_longlong
    lib.rlis_sample_rows.restype = c_int
    lib.rlis_sample_rows.argtypes = [P, L, I, I, P, P, P, I, P, P, P]
    lib.rlis_sample_rows_static.restype = c_int
    lib.rlis_sample_rows_static.argtypes = [P, L, I, I, P, P, P, I, P]
    lib.rlis_sample_rows_static_max_parts.restype = c_int
    lib.rlis_sample_rows_static_max_parts.argtypes = []
    lib.rlis_last_error.restype = ctypes.c_char_p
    lib.rlis_last_error.argtypes = []
    return lib


def _case(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(DEV)
    keys = torch.randint(-2 ** 31, 2 ** 31 - 1, (rows,), generator=g, dtype=torch.int64) \
        .to(torch.int32).to(DEV)
    inv_t = torch.tensor([0.0 if r % 3 == 0 else 1.0 / (0.5 + 0.25 * r) for r in range(rows)],
                         dtype=torch.float32, device=DEV)
    return logits, keys, inv_t


def _both(lib, logits, keys, inv_t, chunks):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    best = torch.empty((rows, chunks), dtype=torch.float32, device=DEV)
    idx = torch.empty((rows, chunks), dtype=torch.int32, device=DEV)
    rc = lib.rlis_sample_rows(logits.data_ptr(), logits.stride(0), rows, vocab, keys.data_ptr(),
                              inv_t.data_ptr(), want.data_ptr(), chunks, best.data_ptr(),
                              idx.data_ptr(), stream)
    assert rc == 0, lib.rlis_last_error()
    got = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    rc = lib.rlis_sample_rows_static(logits.data_ptr(), logits.stride(0), rows, vocab,
                                     keys.data_ptr(), inv_t.data_ptr(), got.data_ptr(), chunks,
                                     stream)
    assert rc == 0, lib.rlis_last_error()
    torch.cuda.synchronize()
    return got.tolist(), want.tolist()


def test_static_sampling_matches_the_allocating_entry_point_twice_in_a_row():
    lib = _library()
    # first call: 48 rows over a vocabulary of 50,021 in 48 chunks
    got, want = _both(lib, *_case(48, 50021, seed=1), chunks=48)
    assert got == want and min(got) >= 0
    # second call, smaller in rows, vocabulary and chunks: stale winners of the first call lie
    # beside and behind what this one writes
    got, want = _both(lib, *_case(5, 3001, seed=2), chunks=3)
    assert got == want and min(got) >= 0 and max(got) < 3001
    # one chunk: no scratch at all
    got, want = _both(lib, *_case(7, 257, seed=3), chunks=1)
    assert got == want
    # and against the plain implementation itself (argmax and Gumbel-max keyed by the row's
    # key, crates/model/src/sampling.rs:45-110), not only against the other entry point
    import plain_llama as plain
    logits, keys, inv_t = _case(6, 1500, seed=5)
    got, _ = _both(lib, logits, keys, inv_t, chunks=4)
    for r in range(6):
        key = int(keys[r]) & 0xFFFFFFFF
        assert got[r] == plain.sample_row(logits[r].cpu(), key, float(inv_t[r])), r


def test_static_sampling_refuses_more_than_its_scratch_holds():
    lib = _library()
    limit = lib.rlis_sample_rows_static_max_parts()
    assert limit == 16384
    rows, chunks = 300, 64                      # 19,200 partial results
    logits, keys, inv_t = _case(rows, 4096, seed=4)
    out = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    rc = lib.rlis_sample_rows_static(logits.data_ptr(), logits.stride(0), rows, 4096,
                                     keys.data_ptr(), inv_t.data_ptr(), out.data_ptr(), chunks,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert b"exceed" in lib.rlis_last_error()
    torch.cuda.synchronize()
    assert out.tolist() == [-7] * rows          # nothing was launched
