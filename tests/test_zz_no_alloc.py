"""The arg-max entry point that allocates nothing (``cw_argmax_static``: its partial results live
in a fixed array inside the library), called through ctypes as a caller outside Python would, and
checked against the ordinary entry point with a workspace: two calls in a row, the second with a
smaller input, so that what the first call left in the array must not show."""

import ctypes
from ctypes import c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256  # CW_ARGMAX_STATIC_MAX_ROWS in csrc/sampling.h


def _library():
    from clockwork_amd.csrc import build

    lib = ctypes.CDLL(str(build.ensure_built("sampling")))
    lib.cw_argmax_chunks.argtypes = [c_int]
    lib.cw_argmax.argtypes = [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_int64, c_void_p]
    lib.cw_argmax_static_init.argtypes = []
    lib.cw_argmax_static.argtypes = [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]
    for name in ("cw_argmax_chunks", "cw_argmax", "cw_argmax_static_init", "cw_argmax_static"):
        getattr(lib, name).restype = c_int
    return lib


def _with_workspace(lib, logits, stream):
    n, V = logits.shape
    chunks = lib.cw_argmax_chunks(V)
    ws = torch.empty(n * chunks * 2, dtype=torch.int32, device=logits.device)
    out = torch.full((n,), -7, dtype=torch.int32, device=logits.device)
    assert lib.cw_argmax(logits.data_ptr(), logits.stride(0), n, V, out.data_ptr(), ws.data_ptr(), ws.numel() * 4, stream) == 0
    return out


def test_argmax_without_allocation_equals_the_one_with_a_workspace():
    lib = _library()
    device = torch.device("cuda", torch.cuda.current_device())
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.cw_argmax_static_init() == 0
    gen = torch.Generator().manual_seed(17)
    # first call: as many rows as the array takes, a vocabulary that fills every chunk (64 of them)
    big = torch.randn(MAX_ROWS, 300_001, generator=gen).to(device)
    big[3, 5] = big[3, 70_000] = 50.0      # equal maxima: the first index wins
    big[4, 299_999] = float("nan")         # a NaN never wins
    big[5] = float("-inf")                 # nothing to choose from: index 0
    # second call: fewer rows, fewer chunks, a row stride wider than the row
    wide = torch.randn(7, 5_000, generator=gen).to(device)
    small = wide[:, :4_097]
    small[2, 4_096] = 40.0                 # the last element, alone in the second chunk
    outputs = []
    for logits in (big, small):
        n, V = logits.shape
        out = torch.full((n,), -7, dtype=torch.int32, device=device)
        torch.cuda.synchronize()
        # neither torch's allocator nor the runtime's (hipMalloc: the device's free memory) is asked
        before = torch.cuda.memory_stats(device)["allocation.all.allocated"], torch.cuda.mem_get_info(device)[0]
        assert lib.cw_argmax_static(logits.data_ptr(), logits.stride(0), n, V, out.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert (torch.cuda.memory_stats(device)["allocation.all.allocated"], torch.cuda.mem_get_info(device)[0]) == before
        outputs.append((out, _with_workspace(lib, logits, stream), logits))
    torch.cuda.synchronize()
    for got, want, logits in outputs:
        assert torch.equal(got.cpu(), want.cpu())
        ref = torch.where(torch.isnan(logits), torch.full_like(logits, float("-inf")), logits).argmax(dim=1)
        assert torch.equal(got.cpu().long(), ref.cpu())
    assert int(outputs[0][0][3]) == 5 and int(outputs[0][0][5]) == 0 and int(outputs[1][0][2]) == 4_096


def test_argmax_without_allocation_inside_a_captured_graph():
    """What the entry point is for: a caller under HIP-graph capture, where an allocation is an
    error. The call is captured (after ``cw_argmax_static_init``, which looks the array up and may
    not run under capture), replayed several times over changing inputs with eager work between
    the replays, and every replay is checked against the ordinary entry point."""
    lib = _library()
    device = torch.device("cuda", torch.cuda.current_device())
    assert lib.cw_argmax_static_init() == 0
    gen = torch.Generator().manual_seed(23)
    logits = torch.randn(9, 70_001, generator=gen).to(device)
    out = torch.full((9,), -7, dtype=torch.int32, device=device)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        code = lib.cw_argmax_static(logits.data_ptr(), logits.stride(0), 9, 70_001, out.data_ptr(),
                                    torch.cuda.current_stream().cuda_stream)
    assert code == 0
    for trial in range(3):
        logits.copy_(torch.randn(9, 70_001, generator=gen))
        logits[trial, 70_000 - trial] = 30.0
        graph.replay()
        torch.cuda.synchronize()
        want = _with_workspace(lib, logits, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want.cpu()) and int(out[trial]) == 70_000 - trial


def test_argmax_without_allocation_refuses_more_rows_than_its_array_holds():
    lib = _library()
    device = torch.device("cuda", torch.cuda.current_device())
    logits = torch.zeros(MAX_ROWS + 1, 8, device=device)
    out = torch.full((MAX_ROWS + 1,), -7, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.cw_argmax_static(logits.data_ptr(), 8, MAX_ROWS + 1, 8, out.data_ptr(), stream) == -4
    assert lib.cw_argmax_static(logits.data_ptr(), 4, 2, 8, out.data_ptr(), stream) == -1  # rows overlap
    torch.cuda.synchronize()
    assert bool((out == -7).all())  # nothing was launched
