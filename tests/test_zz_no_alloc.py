"""The entry point that allocates nothing (`distie_argmax_static`, distie_amd/csrc/no_alloc.h), called
through ctypes and compared with `distie_argmax`, whose scratch the caller allocates."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from distie_amd.csrc import build

    lib = ctypes.CDLL(str(build.ensure("ops")))
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.distie_argmax.argtypes = [P, P, I, I, P, P, P]
    lib.distie_argmax_parts.argtypes = [I, I]
    lib.distie_argmax_static.argtypes = [P, P, I, I, P]
    lib.distie_argmax_static_limits.argtypes = [ctypes.POINTER(I), ctypes.POINTER(I)]
    lib.distie_argmax_static_prepare.argtypes = []
    return lib


def _both(lib, logits):
    """-> (picks of the entry point that allocates nothing, picks of the existing one)"""
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    assert lib.distie_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream) == 0
    want = torch.full((rows,), -9, dtype=torch.int32, device=logits.device)
    parts = lib.distie_argmax_parts(rows, vocab)
    values = torch.empty(rows * parts, dtype=torch.float32, device=logits.device)
    indexes = torch.empty(rows * parts, dtype=torch.int32, device=logits.device)
    assert lib.distie_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, values.data_ptr(), indexes.data_ptr(),
                             stream) == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu(), parts


def test_two_calls_in_a_row_the_second_smaller():
    lib = _library()
    gen = torch.Generator().manual_seed(5)
    first = torch.randn((48, 151_936), generator=gen).cuda()
    # the winner of some rows sits at a piece's edge, and two rows have equal maxima: the lowest index wins
    first[3, 0] = 50.0
    first[4, 151_935] = 50.0
    first[5, 70_000] = first[5, 20_000] = 60.0
    got, want, parts = _both(lib, first)
    assert parts > 1                                  # the scratch was used
    assert torch.equal(got, want)
    assert torch.equal(got.long(), first.argmax(dim=1).cpu())
    assert got[5] == 20_000
    # a smaller input right after: what the first call left in the array must not show
    second = torch.randn((5, 40_000), generator=gen).cuda()
    got, want, parts = _both(lib, second)
    assert parts > 1
    assert torch.equal(got, want)
    assert torch.equal(got.long(), second.argmax(dim=1).cpu())
    # a vocabulary that takes the single-launch path needs no scratch at all
    third = torch.randn((7, 1000), generator=gen).cuda()
    got, want, parts = _both(lib, third)
    assert parts == 1 and torch.equal(got, want)


def test_sizes_beyond_the_maximum_are_refused():
    lib = _library()
    max_rows, max_entries = ctypes.c_int(), ctypes.c_int()
    lib.distie_argmax_static_limits(ctypes.byref(max_rows), ctypes.byref(max_entries))
    assert max_rows.value == 1024 and max_entries.value == 1024
    stream = torch.cuda.current_stream().cuda_stream
    logits = torch.zeros((4, 64), device="cuda")
    out = torch.zeros(4, dtype=torch.int32, device="cuda")
    # refused before anything is launched or read: the row count alone decides
    assert lib.distie_argmax_static(logits.data_ptr(), out.data_ptr(), max_rows.value + 1, 64, stream) == -2
    assert lib.distie_argmax_static(logits.data_ptr(), out.data_ptr(), 4, 0, stream) == -1
    assert lib.distie_argmax_static(logits.data_ptr(), out.data_ptr(), 0, 64, stream) == 0


def test_recorded_into_a_graph_after_the_device_was_prepared():
    """The callers the entry point is for: the array's address is looked up outside the capture
    (`distie_argmax_static_prepare`), the launches are recorded, and every replay picks what the eager entry
    point picks for the logits that lie in the buffer then, with eager work and waits between the replays."""
    lib = _library()
    assert lib.distie_argmax_static_prepare() == 0
    gen = torch.Generator().manual_seed(6)
    logits = torch.randn((24, 151_936), generator=gen).cuda()
    out = torch.full((24,), -7, dtype=torch.int32, device="cuda")
    assert lib.distie_argmax_parts(24, 151_936) > 1
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = lib.distie_argmax_static(logits.data_ptr(), out.data_ptr(), 24, 151_936,
                                          torch.cuda.current_stream().cuda_stream)
    assert status == 0
    for round_ in range(4):
        fresh = torch.randn((24, 151_936), generator=gen)
        fresh[round_, 151_935 - round_] = 40.0
        logits.copy_(fresh.cuda())
        out.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _, want, _ = _both(lib, logits)                 # eager work on the same array between the replays
        assert torch.equal(out.cpu(), want)
        assert torch.equal(out.cpu().long(), fresh.argmax(dim=1))
