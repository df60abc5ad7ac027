"""The arg-max entry point that allocates nothing, called through ctypes as a caller without an
allocator would: its partial results live in an array inside the library's device image.  Checked
against the entry point that takes a workspace, on two calls in a row, the second smaller (the
array then still holds the first call's words)."""

from __future__ import annotations

import ctypes
from ctypes import c_int, c_longlong, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_MAX_ROWS = 1024      # FE_ARGMAX_STATIC_MAX_ROWS of csrc/sample_api.h


def _library() -> ctypes.CDLL:
    from forge_engine_amd.kernels import library

    lib = library.load("sample")
    lib.fe_argmax_rows_static.restype = c_int
    lib.fe_argmax_rows.restype = c_int
    return lib


def _call_static(lib, logits, rows, vocab, out):
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.fe_argmax_rows_static(
        c_void_p(logits.data_ptr()), c_longlong(logits.stride(0)), c_int(rows), c_int(vocab),
        c_void_p(out[0].data_ptr()), c_void_p(out[1].data_ptr()), stream)


def _prime(lib, device) -> None:
    """The first call on a device looks the array's address up (and may make the runtime load the
    library's device image): set-up, done once, before anything is measured or captured."""
    logits = torch.zeros(1, 8, device=device)
    out = torch.zeros((2, 1), dtype=torch.int32, device=device)
    assert _call_static(lib, logits, 1, 8, out) == 0
    torch.cuda.synchronize()


def _static(lib, logits, rows, vocab):
    out = torch.full((2, rows), -7, dtype=torch.int32, device=logits.device)
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated(logits.device)
    reserved = torch.cuda.memory_reserved(logits.device)
    free_before, _ = torch.cuda.mem_get_info(logits.device)
    status = _call_static(lib, logits, rows, vocab, out)
    # the device's own count of free memory did not move (a hipMalloc or hipFree inside the library
    # would move it; torch's counters only see torch's allocator), while the call is queued ...
    assert torch.cuda.mem_get_info(logits.device)[0] == free_before
    torch.cuda.synchronize()
    # ... and after it has run; and torch's allocator saw nothing of the call either
    assert torch.cuda.mem_get_info(logits.device)[0] == free_before
    assert torch.cuda.memory_allocated(logits.device) == allocated
    assert torch.cuda.memory_reserved(logits.device) == reserved
    return status, out


def _with_workspace(lib, logits, rows, vocab):
    out = torch.full((2, rows), -9, dtype=torch.int32, device=logits.device)
    scratch = torch.empty(rows * 32 * 3, dtype=torch.int32, device=logits.device)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.fe_argmax_rows(
        c_void_p(logits.data_ptr()), c_longlong(logits.stride(0)), c_int(rows), c_int(vocab),
        c_void_p(out[0].data_ptr()), c_void_p(out[1].data_ptr()), c_void_p(scratch.data_ptr()), stream)
    return status, out


def test_argmax_without_allocation_equals_the_workspace_entry_point_twice_in_a_row():
    lib = _library()
    device = torch.device("cuda:0")
    _prime(lib, device)
    g = torch.Generator().manual_seed(31)
    first = torch.randn(37, 5003, generator=g).to(device)
    first[3, 17] = float("nan")                      # the status words travel through the array too
    first[5] = float("-inf")
    first[9, 4000:4003] = 50.0                       # equal maxima: the lowest index wins
    second = torch.randn(5, 1201, generator=g).to(device)   # smaller in both directions
    second[2, 1200] = float("inf")
    for logits in (first, second):
        rows, vocab = logits.shape
        status, got = _static(lib, logits, rows, vocab)
        assert status == 0
        status, want = _with_workspace(lib, logits, rows, vocab)
        assert status == 0
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        clean = [r for r in range(rows) if want[1, r] == 0]
        assert got[0, clean].tolist() == logits[clean].argmax(dim=-1).tolist()
    assert got[1].tolist() == [0, 0, 2, 0, 0]
    # as many rows as the array holds, and one more
    most = torch.randn(STATIC_MAX_ROWS + 1, 96, generator=g).to(device)
    status, got = _static(lib, most, STATIC_MAX_ROWS, 96)
    assert status == 0
    torch.cuda.synchronize()
    assert got[0].tolist() == most[:STATIC_MAX_ROWS].argmax(dim=-1).tolist()
    status, got = _static(lib, most, STATIC_MAX_ROWS + 1, 96)
    assert status == 1                                # refused: beyond the array
    torch.cuda.synchronize()
    assert got.eq(-7).all()                           # and nothing ran


def test_argmax_without_allocation_inside_a_captured_graph():
    """What the entry point is for: a call recorded into a HIP graph (the address was looked up by
    an earlier call, outside the capture), replayed with other inputs and with eager work and
    synchronisations between the replays; every replay equals the eager result."""
    lib = _library()
    device = torch.device("cuda:0")
    _prime(lib, device)
    rows, vocab = 19, 3001
    g = torch.Generator().manual_seed(32)
    logits = torch.randn(rows, vocab, generator=g).to(device)
    out = torch.full((2, rows), -7, dtype=torch.int32, device=device)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        assert _call_static(lib, logits, rows, vocab, out) == 0
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert _call_static(lib, logits, rows, vocab, out) == 0
    for replay in range(4):
        fresh = torch.randn(rows, vocab, generator=g)
        fresh[replay, 7:9] = 40.0 + replay           # equal maxima: the lowest index wins
        logits.copy_(fresh.to(device))
        out.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert out[0].tolist() == fresh.argmax(dim=-1).tolist() and out[0, replay] == 7
        assert out[1].eq(0).all()
        # eager work between the replays, through the same array
        status, eager = _static(lib, torch.randn(3, 777, generator=g).to(device), 3, 777)
        assert status == 0
