"""The entry point that allocates nothing, ``pl_argmax_static``, called through ctypes: the greedy
choice over scratch memory that the library owns, against the ordinary entry point ``pl_argmax``
(scratch from the caller), on two calls in a row, the second with a smaller input."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _entry_points():
    from paged_llm_rs_amd import build

    lib = ctypes.CDLL(str(build.build("hip")))
    p, i = ctypes.c_void_p, ctypes.c_int
    lib.pl_argmax_static.argtypes = [p, p, i, i, p]
    lib.pl_argmax_static.restype = i
    lib.pl_argmax.argtypes = [p, p, p, p, i, i, p]
    lib.pl_argmax.restype = i
    lib.pl_last_error.restype = ctypes.c_char_p
    return lib


def _both(lib, logits):
    m, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((m,), -7, dtype=torch.int32, device=DEV)
    assert lib.pl_argmax_static(logits.data_ptr(), got.data_ptr(), m, V, stream) == 0, lib.pl_last_error().decode()
    want = torch.full((m,), -9, dtype=torch.int32, device=DEV)
    scratch_v = torch.empty(m * 64, dtype=torch.float32, device=DEV)
    scratch_i = torch.empty(m * 64, dtype=torch.int32, device=DEV)
    assert lib.pl_argmax(logits.data_ptr(), want.data_ptr(), scratch_v.data_ptr(), scratch_i.data_ptr(), m, V, stream) == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_the_greedy_choice_over_the_librarys_own_scratch_memory():
    lib = _entry_points()
    torch.manual_seed(5)
    # a large call first, then a smaller one (fewer rows and a shorter vocabulary) over what the first left
    first = torch.randn(37, 151936, device=DEV)
    first[3, 150000] = 50.0
    first[4, 7] = first[4, 90001] = 60.0           # the first of two equal maxima wins
    second = torch.randn(5, 1001, device=DEV)
    second[2, 1000] = 40.0
    for logits in (first, second, first[:1].contiguous()):
        got, want = _both(lib, logits)
        assert torch.equal(got, want)
        assert torch.equal(got.long(), torch.argmax(logits, dim=-1).cpu())
    assert int(_both(lib, first)[0][3]) == 150000 and int(_both(lib, first)[0][4]) == 7
    # the most rows it takes, and one more
    full = torch.randn(1024, 300, device=DEV)
    got, want = _both(lib, full)
    assert torch.equal(got, want)
    out = torch.zeros(1025, dtype=torch.int32, device=DEV)
    over = torch.randn(1025, 300, device=DEV)
    assert lib.pl_argmax_static(over.data_ptr(), out.data_ptr(), 1025, 300, torch.cuda.current_stream().cuda_stream) != 0
    assert b"1024" in lib.pl_last_error()
    assert not out.any(), "a refused call launches nothing"


def test_it_allocates_nothing():
    lib = _entry_points()
    logits = torch.randn(8, 5003, device=DEV)
    out = torch.empty(8, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    lib.pl_argmax_static(logits.data_ptr(), out.data_ptr(), 8, 5003, stream)       # the device's address is asked for here
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        assert lib.pl_argmax_static(logits.data_ptr(), out.data_ptr(), 8, 5003, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    assert torch.equal(out.long().cpu(), torch.argmax(logits, dim=-1).cpu())


def test_it_runs_where_allocating_is_an_error():
    """Free memory need not move when a small allocation is made.  A stream that is being captured is a place
    where hipMalloc and hipFree are errors that end the capture: the entry point is recorded there (as one of the
    callers it is for would), and the graph, replayed over other logits, gives what the ordinary entry point gives."""
    lib = _entry_points()
    logits = torch.randn(11, 4099, device=DEV)
    out = torch.full((11,), -3, dtype=torch.int32, device=DEV)
    lib.pl_argmax_static(logits.data_ptr(), out.data_ptr(), 11, 4099, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    out.fill_(-3)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = lib.pl_argmax_static(logits.data_ptr(), out.data_ptr(), 11, 4099, torch.cuda.current_stream().cuda_stream)
    assert status == 0, lib.pl_last_error().decode()
    assert bool((out == -3).all()), "recorded, not run"
    for seed in (1, 2, 3):
        logits.copy_(torch.randn(11, 4099, generator=torch.Generator().manual_seed(seed)))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.long().cpu(), torch.argmax(logits, dim=-1).cpu())
