"""``kvc_argmax_static``: the argmax for callers that cannot allocate.  It is called through
ctypes, as such a caller would, and compared with ``kvc_argmax`` and its caller-given
workspace on two calls in a row, the second with a smaller input (what the first call left
in the static array must not show)."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    from kvcore_amd.ops import library

    return library.load()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _reference(lib, logits: torch.Tensor) -> torch.Tensor:
    """The existing entry point with a workspace of the caller's."""
    S, V = logits.shape
    chunks = -(-V // 8192)
    out = torch.full((S,), -7, dtype=torch.int32, device=DEV)
    part_val = torch.empty(S * chunks, dtype=torch.float32, device=DEV)
    part_idx = torch.empty(S * chunks, dtype=torch.int32, device=DEV)
    code = lib.kvc_argmax(out.data_ptr(), logits.data_ptr(), S, V, logits.stride(0),
                          part_val.data_ptr(), part_idx.data_ptr(), S * chunks, _stream())
    assert code == 0, lib.kvc_last_error()
    return out


def _static(lib, logits: torch.Tensor, out: torch.Tensor) -> int:
    S, V = logits.shape
    return lib.kvc_argmax_static(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(logits.data_ptr()),
                                 S, V, logits.stride(0), ctypes.c_void_p(_stream()))


def _logits(S: int, V: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(S, V, generator=g)
    # the winner of each row in another chunk, and equal maxima whose lowest index must win
    for s in range(S):
        at = (s * 7919 + 13) % V
        x[s, at] = 9.0
        if s % 3 == 0 and at + 8200 < V:
            x[s, at + 8200] = 9.0
    return x.to(DEV)


def test_static_argmax_two_calls_in_a_row(lib):
    big = _logits(37, 128256, seed=1)       # 16 chunks a row
    small = _logits(5, 20000, seed=2)       # 3 chunks a row: reads less of the array than is dirty
    out_big = torch.full((37,), -7, dtype=torch.int32, device=DEV)
    out_small = torch.full((5,), -7, dtype=torch.int32, device=DEV)
    # the first call on a device looks up the array's address (and may load the code object):
    # that is set-up; what is measured is a call after it
    warm = torch.full((5,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, small, warm) == 0, lib.kvc_last_error()
    torch.cuda.synchronize()
    # torch's counters see its own allocator only; the device's free memory sees every
    # hipMalloc of the process, the library's included
    before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    assert _static(lib, big, out_big) == 0, lib.kvc_last_error()
    assert _static(lib, small, out_small) == 0, lib.kvc_last_error()
    torch.cuda.synchronize()
    after = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    assert after == before
    assert torch.equal(out_big, _reference(lib, big))
    assert torch.equal(out_small, _reference(lib, small))
    assert out_big.tolist() == big.cpu().argmax(-1).tolist()
    assert out_small.tolist() == small.cpu().argmax(-1).tolist()
    # and once more the other way round, on the array the small call left
    out_big.fill_(-7)
    assert _static(lib, big, out_big) == 0, lib.kvc_last_error()
    assert torch.equal(out_big, _reference(lib, big))


def test_static_argmax_inside_a_captured_graph(lib):
    """The callers it is for: a stream under capture cannot allocate.  Both calls are recorded
    into one graph (the address was looked up before, outside the capture) and every replay,
    with eager work of the same entry point in between, gives what ``kvc_argmax`` gives."""
    big = _logits(21, 128256, seed=5)
    small = _logits(4, 20000, seed=6)
    out_big = torch.full((21,), -7, dtype=torch.int32, device=DEV)
    out_small = torch.full((4,), -7, dtype=torch.int32, device=DEV)
    other = _logits(9, 50000, seed=7)
    out_other = torch.full((9,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, small, out_small) == 0, lib.kvc_last_error()  # set-up, outside the capture
    want_big, want_small = _reference(lib, big), _reference(lib, small)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            assert _static(lib, big, out_big) == 0, lib.kvc_last_error()
            assert _static(lib, small, out_small) == 0, lib.kvc_last_error()
    for i in range(3):
        out_big.fill_(-7)
        out_small.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_big, want_big) and torch.equal(out_small, want_small), f"replay {i}"
        assert _static(lib, other, out_other) == 0, lib.kvc_last_error()  # dirties the array in between
        torch.cuda.synchronize()
        assert out_other.tolist() == other.cpu().argmax(-1).tolist()


def test_static_argmax_strided_and_short_rows(lib):
    wide = _logits(4, 30000, seed=3)
    view = wide[:, :17000]  # row stride larger than the row
    out = torch.full((4,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, view, out) == 0, lib.kvc_last_error()
    assert out.tolist() == view.cpu().argmax(-1).tolist()
    short = _logits(3, 1000, seed=4)  # one chunk: no partial results at all
    out3 = torch.full((3,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, short, out3) == 0, lib.kvc_last_error()
    assert out3.tolist() == short.cpu().argmax(-1).tolist()


def test_static_argmax_refuses_what_the_array_cannot_hold(lib):
    cap = lib.kvc_argmax_static_capacity()
    assert cap == 16384
    V = 3 * 8192  # 3 chunks a row
    rows = cap // 3 + 1
    logits = torch.zeros(rows, V, device=DEV)
    out = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, logits, out) != 0
    assert b"16384" in lib.kvc_last_error()
    torch.cuda.synchronize()
    assert (out == -7).all()  # nothing was launched
    fits = logits[: cap // 3]
    out2 = torch.full((cap // 3,), -7, dtype=torch.int32, device=DEV)
    assert _static(lib, fits, out2) == 0, lib.kvc_last_error()
    torch.cuda.synchronize()
    assert (out2 == 0).all()  # all equal: the lowest index
