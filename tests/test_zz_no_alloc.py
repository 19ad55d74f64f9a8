"""GPU: ucm_hamming_topk_static (the entry point that allocates nothing) against ucm_hamming_topk
and the CPU checker, bit-exact, through the C ABI.  Two calls in a row share the library's fixed
scratch array; the second one is smaller, so stale cells of the first lie right behind its own.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import make_paged_case
from oracle import c_api

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 4 << 20  # UCM_TOPK_STATIC_SCRATCH_BYTES of include/ucm_hip.h


def _dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.cuda()


def _call(static, q, kc, table, lens, k, flags, sink=0, recent=0):
    """One call of either entry point with raw pointers; returns (idx, score) as numpy."""
    from ucm_amd import _lib

    L = _lib.lib()
    B, Hq, Wd = q.shape
    NB, BS, Hkv, _ = kc.shape
    mb = table.shape[1]
    Ho = 1 if flags & _lib.TOPK_REDUCE_HEADS else Hkv
    dq, dk, dt, dl = _dev(q.view(np.int32)), _dev(kc.view(np.int32)), _dev(table), _dev(lens)
    idx = torch.full((B, Ho, k), -7, dtype=torch.int32, device="cuda")
    sc = torch.full((B, Ho, k), -7, dtype=torch.int32, device="cuda")
    st = _lib.stream_ptr(dq.device)
    head = (dq.data_ptr(), Hq * Wd, Wd, dk.data_ptr(), NB, BS, Hkv, Wd, BS * Hkv * Wd, Hkv * Wd, Wd,
            dt.data_ptr(), mb, mb, dl.data_ptr(), B, Hq, k, sink, recent, flags,
            idx.data_ptr(), sc.data_ptr())
    if static:
        rc = L.ucm_hamming_topk_static(*head, st)
    else:
        n = L.ucm_hamming_topk_workspace_bytes(B, Hkv, mb)
        ws = torch.empty(n, dtype=torch.uint8, device="cuda")
        rc = L.ucm_hamming_topk(*head, ws.data_ptr(), n, st)
    _lib.check(rc)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), sc.cpu().numpy()


# (seed, B, Hq, Hkv, Wd, BS, lens, k, flags): a larger call, then a smaller one
CALLS = [
    (11, 4, 32, 8, 4, 128, [32768, 20001, 128, 9000], 64, 0),
    (12, 2, 32, 8, 4, 128, [700, 3000], 5, 0),
]
MLA_CALLS = [
    (13, 3, 128, 1, 8, 64, [65536, 40000, 77], 128, 0),       # bit planes live in the scratch
    (14, 2, 128, 1, 8, 64, [4096, 640], 16, 2),               # physical ids
]
REDUCED_CALLS = [
    (15, 3, 16, 4, 3, 16, [5000, 333, 4097], 24, 1 | 2),      # general kernel, head-reduced rows
    (16, 1, 16, 4, 3, 16, [1000], 7, 1),
]


@pytest.mark.parametrize("calls", [CALLS, MLA_CALLS, REDUCED_CALLS], ids=["gqa", "planes", "reduced"])
def test_static_entry_point_matches_the_workspace_one(calls):
    for seed, B, Hq, Hkv, Wd, BS, lens, k, flags in calls:
        q, kc, table, lens = make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens)
        ref_i, ref_s = _call(False, q, kc, table, lens, k, flags)
        got_i, got_s = _call(True, q, kc, table, lens, k, flags)
        assert np.array_equal(got_i, ref_i)
        assert np.array_equal(got_s, ref_s)
        oi, os_ = c_api.hamming_topk(q, kc, table, lens, k, 0, 0, flags)
        assert np.array_equal(got_i, oi)
        assert np.array_equal(got_s, os_)


def test_static_entry_point_rejects_shapes_beyond_its_scratch():
    from ucm_amd import _lib

    L = _lib.lib()
    B, Hkv, mb = 64, 8, 4096  # 8 MiB of block scores alone
    assert L.ucm_hamming_topk_workspace_bytes(B, Hkv, mb) > SCRATCH_BYTES
    q, kc, table, lens = make_paged_case(17, 1, 32, 8, 4, 128, [256])
    dq, dk, dl = _dev(q.view(np.int32)), _dev(kc.view(np.int32)), _dev(lens)
    out = torch.empty((B, Hkv, 4), dtype=torch.int32, device="cuda")
    rc = L.ucm_hamming_topk_static(dq.data_ptr(), 128, 4, dk.data_ptr(), kc.shape[0], 128, 8, 4,
                                   128 * 32, 32, 4, None, 0, mb, dl.data_ptr(), B, 32, 4, 0, 0, 0,
                                   out.data_ptr(), None, _lib.stream_ptr(dq.device))
    assert rc == _lib.UCM_EPARAM
    assert b"scratch" in L.ucm_last_error()


def test_static_entry_point_allocates_nothing_and_replays_in_a_graph():
    """What the entry point exists for: after a first call on the device (which looks up the scratch
    array's address) a call takes no device memory - free memory is the same before and after -
    and can be captured into a HIP graph whose replays, with eager work and synchronisations in
    between, all give the workspace entry point's result."""
    from ucm_amd import _lib

    L = _lib.lib()
    seed, B, Hq, Hkv, Wd, BS, lens, k, flags = MLA_CALLS[0]
    q, kc, table, lens = make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens)
    ref_i, ref_s = _call(False, q, kc, table, lens, k, flags)
    _call(True, q, kc, table, lens, k, flags)  # warm-up: address look-up, code object load

    NB, mb = kc.shape[0], table.shape[1]
    dq, dk, dt, dl = _dev(q.view(np.int32)), _dev(kc.view(np.int32)), _dev(table), _dev(lens)
    idx = torch.full((B, 1, k), -7, dtype=torch.int32, device="cuda")
    sc = torch.full((B, 1, k), -7, dtype=torch.int32, device="cuda")

    def launch(stream_ptr):
        _lib.check(L.ucm_hamming_topk_static(
            dq.data_ptr(), Hq * Wd, Wd, dk.data_ptr(), NB, BS, Hkv, Wd, BS * Hkv * Wd, Hkv * Wd, Wd,
            dt.data_ptr(), mb, mb, dl.data_ptr(), B, Hq, k, 0, 0, flags, idx.data_ptr(), sc.data_ptr(),
            stream_ptr))

    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    launch(_lib.stream_ptr(dq.device))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert np.array_equal(idx.cpu().numpy(), ref_i) and np.array_equal(sc.cpu().numpy(), ref_s)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launch(side.cuda_stream)
    for rep in range(3):
        idx.fill_(-7)
        sc.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(idx.cpu().numpy(), ref_i), rep
        assert np.array_equal(sc.cpu().numpy(), ref_s), rep
        # eager work of the program's own between the replays
        got_i, _ = _call(True, q, kc, table, lens, k, flags)
        assert np.array_equal(got_i, ref_i)
