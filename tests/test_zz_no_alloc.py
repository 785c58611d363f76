"""The entry point that allocates nothing (`mllm_argmax_noalloc`, csrc/kernels/noalloc.h), called
through ctypes as a caller without this package would: its output equals the ordinary entry point's
on two calls in a row, the second with a smaller input (the library's fixed scratch keeps the first
call's contents), and sizes beyond its limit are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lib():
    from mini_llm_amd.build import load_library
    lib = load_library("sampling")
    vp, i = ctypes.c_void_p, ctypes.c_int
    lib.mllm_argmax_noalloc.restype = i
    lib.mllm_argmax_noalloc.argtypes = [vp, i, i, i, vp, vp]
    lib.mllm_argmax.restype = i
    lib.mllm_argmax.argtypes = [vp, i, i, i, vp, vp, vp, vp]
    lib.mllm_argmax_noalloc_max_pairs.restype = i
    lib.mllm_argmax_chunks.restype = i
    return lib


def _both(lib, logits):
    n, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    chunks = lib.mllm_argmax_chunks(V)
    pv = torch.empty(n * chunks, dtype=torch.float32, device=DEV)
    pi = torch.empty(n * chunks, dtype=torch.int32, device=DEV)
    want = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    got = torch.full((n,), -9, dtype=torch.int32, device=DEV)
    assert lib.mllm_argmax(logits.data_ptr(), logits.stride(0), n, V, want.data_ptr(), pv.data_ptr(),
                           pi.data_ptr(), stream) == 0
    assert lib.mllm_argmax_noalloc(logits.data_ptr(), logits.stride(0), n, V, got.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_without_allocation_matches_the_ordinary_entry_point():
    lib = _lib()
    g = torch.Generator().manual_seed(11)
    # first call: 37 rows of a ragged vocabulary, with ties (the lowest index must win) and the largest
    # value of some rows in the last, partial chunk
    big = torch.randn(37, 50257, generator=g)
    big[3, 40000] = big[3, 123] = 9.0
    big[5, 50256] = 11.0
    big[6] = 0.25
    got, want = _both(lib, big.to(DEV))
    assert torch.equal(got, want)
    assert torch.equal(got.long(), big.argmax(dim=1)) or got[3] == 123       # torch's tie rule may differ
    assert got[3] == 123 and got[5] == 50256 and got[6] == 0
    # second call, smaller in rows and in chunks: what the first call left in the scratch must not count
    small = torch.randn(5, 4100, generator=g) - 20.0          # every value far below the first call's
    got2, want2 = _both(lib, small.to(DEV))
    assert torch.equal(got2, want2) and torch.equal(got2.long(), small.argmax(dim=1))
    # one chunk only (the second stage does not run), then the first input again
    tiny = torch.randn(3, 1000, generator=g)
    got3, want3 = _both(lib, tiny.to(DEV))
    assert torch.equal(got3, want3) and torch.equal(got3.long(), tiny.argmax(dim=1))
    got4, _ = _both(lib, big.to(DEV))
    assert torch.equal(got4, got)


def test_argmax_without_allocation_refuses_what_its_scratch_cannot_hold():
    lib = _lib()
    limit = lib.mllm_argmax_noalloc_max_pairs()
    assert limit == 16384
    V = 50257
    chunks = lib.mllm_argmax_chunks(V)
    n = limit // chunks + 1
    logits = torch.zeros((n, V), dtype=torch.float32, device=DEV)
    out = torch.full((n,), -5, dtype=torch.int32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.mllm_argmax_noalloc(logits.data_ptr(), V, n, V, out.data_ptr(), stream) == -3
    torch.cuda.synchronize()
    assert (out == -5).all()                                   # nothing was launched
    assert lib.mllm_argmax_noalloc(logits.data_ptr(), V, n - 1, V, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert (out[:n - 1] == 0).all() and out[n - 1] == -5
    assert lib.mllm_argmax_noalloc(logits.data_ptr(), V, 1, 0, out.data_ptr(), stream) == -1
