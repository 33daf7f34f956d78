"""The arg-max entry point that allocates nothing (``ls_argmax_static``), called through
ctypes as a caller without an allocator would, against ``ls_argmax`` with a scratch buffer
the caller brings: two calls in a row, the second with a smaller input, so that what the
first call left in the library's static scratch array cannot leak into the second."""

from __future__ import annotations

import ctypes
from ctypes import c_int, c_long, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_PAIRS = 16384      # LS_ARGMAX_STATIC_PAIRS of csrc/core_api.h


def core_library():
    from lockstep_amd.ops import build

    lib = ctypes.CDLL(str(build.build_core()))
    lib.ls_last_error.restype = ctypes.c_char_p
    for fn in (lib.ls_argmax, lib.ls_argmax_static, lib.ls_argmax_chunks):
        fn.restype = c_int
    return lib


def stream_pointer() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def with_scratch(lib, x: torch.Tensor) -> torch.Tensor:
    """The existing entry point, with a scratch buffer allocated here."""
    rows, width = x.shape
    chunks = lib.ls_argmax_chunks(c_int(width))
    scratch = torch.empty(max(1, 2 * rows * chunks), dtype=torch.int32, device=x.device)
    out = torch.full((rows,), -1, dtype=torch.int32, device=x.device)
    code = lib.ls_argmax(c_void_p(x.data_ptr()), c_void_p(out.data_ptr()), c_int(rows), c_int(width),
                         c_long(x.stride(0)), c_void_p(scratch.data_ptr()), c_long(scratch.numel()), stream_pointer())
    assert code == 0, lib.ls_last_error().decode()
    return out


def without_allocation(lib, x: torch.Tensor, out: torch.Tensor) -> int:
    rows, width = x.shape
    return lib.ls_argmax_static(c_void_p(x.data_ptr()), c_void_p(out.data_ptr()), c_int(rows), c_int(width),
                                c_long(x.stride(0)), stream_pointer())


def logits_with_ties(rows: int, width: int, seed: int) -> torch.Tensor:
    """Random rows whose maximum occurs several times, in different chunks, so that the lowest
    index has to win across the chunks' partial results."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, width, generator=g)
    for r in range(rows):
        at = torch.randint(0, width, (3,), generator=g)
        x[r, at] = 9.0 + r
    return x.cuda()


def test_two_calls_in_a_row_the_second_smaller():
    lib = core_library()
    torch.cuda.set_device(0)
    # inputs, outputs and the reference's scratch are allocated before the calls under test
    first = logits_with_ties(37, 151936, seed=1)          # 38 chunks a row
    second = logits_with_ties(5, 20000, seed=2)           # 5 chunks a row: fewer rows, fewer chunks
    third = logits_with_ties(3, 1000, seed=3)             # one chunk: the scratch array is not used
    outs = [torch.full((x.shape[0],), -1, dtype=torch.int32, device="cuda") for x in (first, second, third)]
    want = [with_scratch(lib, x) for x in (first, second, third)]
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated()
    for x, out in zip((first, second, third), outs):
        code = without_allocation(lib, x, out)
        assert code == 0, lib.ls_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held
    for x, out, ref in zip((first, second, third), outs, want):
        assert torch.equal(out, ref)
        assert torch.equal(out.long().cpu(), torch.stack([(row == row.max()).nonzero()[0, 0] for row in x.cpu()]))


def test_the_static_scratch_keeps_nothing_a_later_call_reads():
    """A wide call leaves large winners in the array; a narrower call over small values must
    not see them."""
    lib = core_library()
    big = torch.full((64, 100000), 50.0, device="cuda")
    small = -torch.rand(64, 9000, device="cuda") - 1.0
    out_big = torch.empty(64, dtype=torch.int32, device="cuda")
    out_small = torch.empty(64, dtype=torch.int32, device="cuda")
    want = with_scratch(lib, small)
    assert without_allocation(lib, big, out_big) == 0
    assert without_allocation(lib, small, out_small) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_big, torch.zeros_like(out_big))       # all equal: the lowest index
    assert torch.equal(out_small, want)
    assert torch.equal(out_small.long(), small.argmax(dim=1))


def test_sizes_beyond_the_array_are_refused_and_nothing_runs():
    lib = core_library()
    chunks = lib.ls_argmax_chunks(c_int(151936))
    rows = STATIC_PAIRS // chunks + 1
    x = torch.zeros((rows, 151936), device="cuda")
    out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    assert without_allocation(lib, x, out) != 0
    message = lib.ls_last_error().decode()
    assert "static array holds" in message and str(STATIC_PAIRS) in message
    torch.cuda.synchronize()
    assert bool((out == -7).all())
    # the largest size that fits does run
    fits = x[: STATIC_PAIRS // chunks]
    assert without_allocation(lib, fits, out[: fits.shape[0]]) == 0
    torch.cuda.synchronize()
    assert bool((out[: fits.shape[0]] == 0).all())
