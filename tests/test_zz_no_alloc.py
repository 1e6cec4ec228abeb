"""The sampling entry point that allocates nothing, against the one that takes a workspace.

``sia_sample_static`` keeps its histograms in a fixed array inside the library, which every call on a GPU shares
and which holds the last call's contents.  It is called through ``ctypes`` twice in a row, the second time with
fewer rows and a smaller vocabulary, and must give the tokens of ``sia_sample`` on a fresh zeroed workspace both
times; too many rows are refused.
"""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
REFUSED = 10001


def _library():
    from simple_inference_amd.kernels import build
    lib = build.load_library("core")
    p, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    lib.sia_sample.argtypes = [p, p, p, p, p, p, p, i, i, i, p]
    lib.sia_sample.restype = i
    lib.sia_sample_static.argtypes = [p, p, p, p, p, p, i, i, i, p]
    lib.sia_sample_static.restype = i
    lib.sia_sample_static_max_rows.argtypes = []
    lib.sia_sample_static_max_rows.restype = i
    lib.sia_sample_workspace_bytes.argtypes = [i]
    lib.sia_sample_workspace_bytes.restype = ctypes.c_longlong
    return lib


def _case(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 2.0).to(DEV)
    # greedy rows beside every mix of filters, so that each launch of the series runs and some rows skip it
    temperature = torch.tensor([(0.0, 1.0, 0.7, 1.3, 0.5)[r % 5] for r in range(rows)], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([(0, 5, 0, 50, 3)[(r // 2) % 5] for r in range(rows)], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([(1.0, 0.9, 0.5, 1.0, 0.3)[(r // 3) % 5] for r in range(rows)], dtype=torch.float32, device=DEV)
    uniform = torch.rand(rows, generator=g).to(DEV)
    return logits, temperature, top_k, top_p, uniform


def _both(lib, rows, vocab, seed, filters=7):
    logits, temperature, top_k, top_p, uniform = _case(rows, vocab, seed)
    stream = torch.cuda.current_stream().cuda_stream
    ptr = lambda t: t.data_ptr()
    want = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    workspace = torch.zeros(lib.sia_sample_workspace_bytes(rows), dtype=torch.uint8, device=DEV)
    assert lib.sia_sample(ptr(logits), ptr(temperature), ptr(top_k), ptr(top_p), ptr(uniform), ptr(want),
                          ptr(workspace), rows, vocab, filters, stream) == 0
    got = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    assert lib.sia_sample_static(ptr(logits), ptr(temperature), ptr(top_k), ptr(top_p), ptr(uniform), ptr(got),
                                 rows, vocab, filters, stream) == 0
    torch.cuda.synchronize()
    assert all(0 <= t < vocab for t in want.tolist())
    return got.tolist(), want.tolist()


def test_two_calls_in_a_row_the_second_smaller_match_the_entry_point_with_a_workspace():
    lib = _library()
    got, want = _both(lib, rows=11, vocab=5003, seed=1)
    assert got == want
    got, want = _both(lib, rows=4, vocab=331, seed=2)     # what the first call left in the array must not show
    assert got == want
    got, want = _both(lib, rows=lib.sia_sample_static_max_rows(), vocab=1000, seed=3)   # the most it takes
    assert got == want
    got, want = _both(lib, rows=3, vocab=777, seed=4, filters=0)   # argmax only: nothing is cleared or read
    assert got == want


def test_more_rows_than_the_array_holds_are_refused():
    lib = _library()
    rows = lib.sia_sample_static_max_rows() + 1
    logits, temperature, top_k, top_p, uniform = _case(rows, 64, seed=5)
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    code = lib.sia_sample_static(logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                                 uniform.data_ptr(), out.data_ptr(), rows, 64, 7,
                                 torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert code == REFUSED and out.tolist() == [-1] * rows


def test_recorded_into_a_graph_after_the_address_was_looked_up_outside_it():
    """The look-up of the array's address is no stream operation: ``sia_sample_static_init`` does it before the
    recording starts, and the recorded call then only launches kernels.  The graph is replayed several times on
    new inputs, with eager work and waits between the replays, and every replay gives the eager call's tokens."""
    lib = _library()
    lib.sia_sample_static_init.argtypes, lib.sia_sample_static_init.restype = [], ctypes.c_int
    assert lib.sia_sample_static_init() == 0
    rows, vocab = 6, 4099
    logits, temperature, top_k, top_p, uniform = _case(rows, vocab, seed=20)
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    ptr = lambda t: t.data_ptr()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            code = lib.sia_sample_static(ptr(logits), ptr(temperature), ptr(top_k), ptr(top_p), ptr(uniform), ptr(out),
                                         rows, vocab, 7, torch.cuda.current_stream().cuda_stream)
    assert code == 0
    torch.cuda.current_stream().wait_stream(side)
    for seed in (21, 22, 23):
        fresh = _case(rows, vocab, seed)
        for dst, src in zip((logits, temperature, top_k, top_p, uniform), fresh):
            dst.copy_(src)
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        got = out.tolist()
        want = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        workspace = torch.zeros(lib.sia_sample_workspace_bytes(rows), dtype=torch.uint8, device=DEV)
        assert lib.sia_sample(ptr(logits), ptr(temperature), ptr(top_k), ptr(top_p), ptr(uniform), ptr(want),
                              ptr(workspace), rows, vocab, 7, torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        assert got == want.tolist(), seed
