"""GPU test of ps_overflow_scan_chunks_noalloc, the one entry point that allocates nothing: its partial results live
in a file-scope device array inside the library.  Checked against ps_overflow_scan_chunks (the same probe with a
caller-allocated ps_step_state) on two calls in a row, the second with a smaller input, so that whatever the first
call left in the scratch array would show."""
import ctypes

import numpy as np
import pytest
import torch

import patrickstar_amd as ps
from patrickstar_amd import _lib

pytestmark = pytest.mark.gpu


def _chunks(n_chunks, n, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    slab = (torch.randn(n_chunks * (n + 8), device="cuda", generator=g) * 300).half()
    rows = [[16, 16, 16, slab[c * (n + 8):].data_ptr()] for c in range(n_chunks)]  # fp32 / m / v are never read
    return slab, _lib.chunk_array(rows)


def _existing(table, n_chunks, n):
    s = ps.DynamicLossScaler(init_scale=2)
    s.materialize("cuda:0")
    _lib.check(_lib.load().ps_overflow_scan_chunks(table, n_chunks, n, None, s.state_ptr, _lib.current_stream_handle()), "scan")
    return int(s.overflow_flag)


def _noalloc(table, n_chunks, n, flag):
    _lib.check(
        _lib.load().ps_overflow_scan_chunks_noalloc(table, n_chunks, n, flag.data_ptr(), _lib.current_stream_handle()),
        "ps_overflow_scan_chunks_noalloc",
    )


def test_two_calls_in_a_row_match_the_allocating_entry_point():
    lib = _lib.load()
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    # first call: 70 chunks (two launches of the first kernel) of a ragged length, an inf in the last element of the
    # last chunk -> set
    n_big, c_big = 8192 * 5 + 77, 70
    slab, table = _chunks(c_big, n_big, seed=1)
    assert _existing(table, c_big, n_big) == 0
    _noalloc(table, c_big, n_big, flag)
    assert int(flag.item()) == 0
    slab[(c_big - 1) * (n_big + 8) + n_big - 1] = float("inf")
    assert _existing(table, c_big, n_big) == 1
    _noalloc(table, c_big, n_big, flag)
    assert int(flag.item()) == 1
    # second call: smaller and clean; the scratch array still holds the hit of the first call beyond (and inside) the
    # words this call uses, and must not leak into the answer
    flag.zero_()
    n_small, c_small = 8192 + 3, 3
    slab2, table2 = _chunks(c_small, n_small, seed=2)
    assert _existing(table2, c_small, n_small) == 0
    _noalloc(table2, c_small, n_small, flag)
    assert int(flag.item()) == 0
    # the flag is sticky: a clean probe does not clear a set flag; every position and value is found
    for pos, val in [((0, 0), float("nan")), ((1, 8191), float("-inf")), ((2, n_small - 1), float("inf")), ((1, 8192), float("nan"))]:
        slab2_poisoned = slab2.clone()
        rows = [[16, 16, 16, slab2_poisoned[c * (n_small + 8):].data_ptr()] for c in range(c_small)]
        slab2_poisoned[pos[0] * (n_small + 8) + pos[1]] = val
        t = _lib.chunk_array(rows)
        flag.zero_()
        _noalloc(t, c_small, n_small, flag)
        assert int(flag.item()) == _existing(t, c_small, n_small) == 1, (pos, val)
        _noalloc(table2, c_small, n_small, flag)
        assert int(flag.item()) == 1
    # the gap between chunks is not looked at
    slab2[n_small] = float("inf")
    flag.zero_()
    _noalloc(table2, c_small, n_small, flag)
    assert int(flag.item()) == _existing(table2, c_small, n_small) == 0


def test_limits_and_argument_checks():
    lib = _lib.load()
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    slab, table = _chunks(3, 100, seed=3)  # three descriptors: no call below names more chunks than the array holds
    s = _lib.current_stream_handle()
    E = _lib.PS_ERR_BAD_ARG
    assert lib.ps_overflow_scan_chunks_noalloc(table, 2, 100, None, s) == E
    assert lib.ps_overflow_scan_chunks_noalloc(None, 2, 100, flag.data_ptr(), s) == E
    assert lib.ps_overflow_scan_chunks_noalloc(table, 0, 100, flag.data_ptr(), s) == 0
    assert lib.ps_overflow_scan_chunks_noalloc(table, 2, 0, flag.data_ptr(), s) == 0
    # Sizes beyond the scratch array are rejected before anything is queued (the buffers here are tiny: a call that
    # got through would read far out of bounds).  2^32 elements are 2^19 tiles of 8192: two such chunks fill the 2^20
    # words exactly, so the first size that must be refused is three of them; one chunk of 2^34 is too long alone.
    assert lib.ps_overflow_scan_chunks_noalloc(table, 3, 2**32, flag.data_ptr(), s) == E
    assert b"scratch words" in lib.ps_last_error()
    assert lib.ps_overflow_scan_chunks_noalloc(table, 2, 2**32 + 1, flag.data_ptr(), s) == E
    assert lib.ps_overflow_scan_chunks_noalloc(table, 1, 2**34, flag.data_ptr(), s) == E
    torch.cuda.synchronize()
    assert int(flag.item()) == 0


def test_full_size_probe_matches_the_atomic_form():
    """24 chunks of 64 Mi elements (196,608 scratch words): same answer as ps_overflow_scan_chunks."""
    n, c = 64 * 1024 * 1024, 24
    slab = torch.zeros(c * n, dtype=torch.half, device="cuda")
    table = _lib.chunk_array([[16, 16, 16, slab[k * n:].data_ptr()] for k in range(c)])
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    _noalloc(table, c, n, flag)
    assert int(flag.item()) == _existing(table, c, n) == 0
    slab[17 * n + 12345] = float("nan")
    _noalloc(table, c, n, flag)
    assert int(flag.item()) == _existing(table, c, n) == 1


def test_probe_replays_from_a_hip_graph():
    """What the entry point is for: a caller under stream capture.  The two launches are captured once (after one
    eager call, which resolves the scratch array's address on this GPU) and replayed over changing data, with eager
    work and synchronisation between the replays; every replay must give the allocating entry point's answer."""
    n, c = 8192 * 3 + 5, 66  # two launches of the first kernel
    slab, table = _chunks(c, n, seed=5)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    _noalloc(table, c, n, flag)  # eager
    assert int(flag.item()) == 0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _noalloc(table, c, n, flag)
    clean = slab.clone()
    for it, (chunk, pos, val) in enumerate([(None, 0, 0.0), (65, n - 1, float("inf")), (None, 0, 0.0), (0, 0, float("nan")),
                                            (33, 8192, float("-inf")), (None, 0, 0.0)]):
        slab.copy_(clean)
        if chunk is not None:
            slab[chunk * (n + 8) + pos] = val
        flag.zero_()
        graph.replay()
        torch.cuda.synchronize()
        want = _existing(table, c, n)
        assert want == (chunk is not None)
        assert int(flag.item()) == want, (it, chunk, pos, val)
