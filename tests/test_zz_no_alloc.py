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


def _static(lib, logits, rows, vocab):
    out = torch.full((2, rows), -7, dtype=torch.int32, device=logits.device)
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated(logits.device)
    reserved = torch.cuda.memory_reserved(logits.device)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.fe_argmax_rows_static(
        c_void_p(logits.data_ptr()), c_longlong(logits.stride(0)), c_int(rows), c_int(vocab),
        c_void_p(out[0].data_ptr()), c_void_p(out[1].data_ptr()), stream)
    # torch's allocator saw nothing of the call
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
