"""GPU: top-k calls in flight on two streams at once do not share scratch memory.

The retrieval worker scores on its own side stream while the plugin-side operator runs on the
current stream; both use the host mirror's cached workspace, which is kept per (device, stream).
"""
import numpy as np
import pytest
import torch

from helpers import make_paged_case, rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu


def _dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.cuda()


def test_side_stream_worker_beside_main_stream_topk():
    from ucm_amd.sparse import hamming_topk
    from ucm_amd.sparse.retrieval_worker import HashRetrievalWorkerBackend

    rng = rng_for(4242)
    # worker side: 4096 blocks of 128 tokens x 16-byte codes, two alternating query batches
    data = rng.integers(0, 256, size=(4096, 128, 16), dtype=np.uint8)
    worker_cases = []
    for B, n in ((6, 3000), (3, 1200)):
        query = rng.integers(0, 256, size=(B, 16), dtype=np.uint8)
        indexes = np.full((B, n), -1, np.int32)
        for b in range(B):
            m = int(rng.integers(n // 2, n + 1))
            indexes[b, :m] = rng.choice(4096, size=m, replace=False)
        k = 40
        oi, od, on = c_api.hash_retrieval(data, query, indexes, k)
        worker_cases.append((query, indexes, k, oi, od, on))
    be = HashRetrievalWorkerBackend(data)

    # main stream: two alternating GQA shapes (the larger one regrows the cached scratch)
    main_cases = []
    for seed, B, lens, k in ((1, 8, [16384, 9000, 128, 16000, 7777, 16384, 300, 12000], 32),
                             (2, 16, [32768] * 15 + [20000], 64)):
        q, kc, table, lens = make_paged_case(seed, B, 32, 8, 4, 128, lens)
        oi, os_ = c_api.hamming_topk(q, kc, table, lens, k)
        main_cases.append((_dev(q.view(np.int32)), _dev(kc.view(np.int32)), _dev(table), _dev(lens), k, oi, os_))

    pending, main_out = [], []
    for it in range(300):
        wq, wi, wk, *_ = worker_cases[it % 2]
        pending.append((it % 2, be.submit(torch.from_numpy(wq), wk, wi)))
        dq, dk, dt, dl, k, *_ = main_cases[(it // 3) % 2]
        idx, sc = hamming_topk(dq, dk, dt, dl, k)
        main_out.append(((it // 3) % 2, idx.clone(), sc.clone()))
        if len(pending) >= 8:  # keep a few worker requests in flight
            c, rid = pending.pop(0)
            be.wait(rid)
            res = be.get_result(rid)
            _, _, _, oi, od, on = worker_cases[c]
            for r in range(oi.shape[0]):
                kk = int(on[r])
                assert np.array_equal(res["indices"][r, :kk], oi[r, :kk]), (it, r)
                assert np.array_equal(res["scores"][r, :kk], od[r, :kk]), (it, r)
    torch.cuda.synchronize()
    for c, rid in pending:
        be.wait(rid)
        res = be.get_result(rid)
        _, _, _, oi, od, on = worker_cases[c]
        for r in range(oi.shape[0]):
            kk = int(on[r])
            assert np.array_equal(res["indices"][r, :kk], oi[r, :kk])
            assert np.array_equal(res["scores"][r, :kk], od[r, :kk])
    for c, idx, sc in main_out:
        assert np.array_equal(idx.cpu().numpy(), main_cases[c][5])
        assert np.array_equal(sc.cpu().numpy(), main_cases[c][6])
