"""GPU parity: KVStar block retrieval (ucm_kvstar_topk through the kvstar_retrieve mirror)
against the CPU checker.

Tolerance: block scores are sums of fp32 softmax probabilities; the GPU adds the q.k partial
products and the exponentials in a different order than the checker's sequential loops, and its
expf differs from libm's by a few ulp.  Scores must agree within 2e-5 relative + 1e-7 absolute,
and where the returned block numbers differ the two blocks' checker scores must differ by less
than that tolerance (a tie within rounding).
"""
import numpy as np
import pytest
import torch

from oracle import brute, c_api
from ucm_amd.sparse import kvstar_retrieve

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-5, 1e-7


def make(seed, X, Hq, Hkv, d, n, M, scale=0.5, d_orig=None):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((X, Hq, d_orig or d)) * scale).astype(np.float16)
    k = (rng.standard_normal((n, M, Hkv, d)) * scale).astype(np.float16)
    return q, k


def run_gpu(q, k, pr, topk):
    dev = torch.device("cuda:0")
    idx, sc = kvstar_retrieve.kvstar_topk(
        torch.from_numpy(q).to(dev), torch.from_numpy(k).to(dev),
        torch.from_numpy(pr).to(dev) if pr is not None else None, topk)
    torch.cuda.synchronize()
    return idx.cpu().numpy().astype(np.int64), sc.cpu().numpy()


def check(q, k, pr, topk):
    gi, gs = run_gpu(q, k, pr, topk)
    oi, osc, allsc = c_api.kvstar_topk(q, k, topk, pr)
    assert gi.shape == oi.shape
    tol = ATOL + RTOL * np.abs(osc)
    assert np.all(np.abs(gs - osc) <= tol), (gs, osc)
    assert np.all(np.diff(gs) <= 0)
    assert len(set(gi.tolist())) == gi.size
    for t in np.nonzero(gi != oi)[0]:
        assert abs(allsc[gi[t]] - allsc[oi[t]]) <= 2 * tol[t]
    # the returned score is the score of the returned block
    assert np.all(np.abs(gs - allsc[gi]) <= ATOL + RTOL * np.abs(allsc[gi]))


@pytest.mark.parametrize("X,Hq,Hkv,d,n,M,topk", [
    (1, 4, 4, 16, 7, 1, 3),        # MHA, one representative per block
    (3, 8, 2, 32, 24, 4, 5),       # GQA 4:1
    (8, 32, 8, 128, 100, 2, 16),   # Llama-like heads
    (5, 6, 3, 20, 40, 3, 8),       # head dim not a multiple of 8: scalar K loads
    (2, 4, 1, 64, 300, 1, 300),    # MQA, every block returned
    (17, 8, 8, 128, 513, 2, 64),   # more than one row tile, blocks past one workgroup
    (1, 1, 1, 8, 1, 1, 1),         # smallest problem
    (20, 8, 2, 32, 70, 3, 9),      # 80 query rows per KV head: three row tiles, ragged last tiles
    (3, 4, 2, 48, 33, 1, 5),       # three k-steps, one representative past a 32-wide tile
])
def test_matches_checker(X, Hq, Hkv, d, n, M, topk):
    q, k = make(X * 1000 + n, X, Hq, Hkv, d, n, M)
    check(q, k, None, topk)


def test_sharp_softmax():
    # larger logits: a few representatives take most of the mass
    q, k = make(11, 4, 8, 4, 64, 200, 2, scale=1.5)
    check(q, k, None, 10)


def test_channel_pruning():
    rng = np.random.default_rng(12)
    Hkv, d_orig, d = 2, 128, 96
    q, k = make(12, 4, 8, Hkv, d, 64, 2, d_orig=d_orig)
    pr = np.stack([np.sort(rng.permutation(d_orig)[:d]) for _ in range(Hkv)]).astype(np.int64)
    check(q, k, pr, 12)


def test_against_float64_formulation_at_llama_shape():
    # a size the sequential checker would take long on: 8 query tokens x 32 heads against 4096
    # blocks x 2 representatives, compared with the float64 library formulation
    q, k = make(13, 8, 32, 8, 128, 4096, 2, scale=0.3)
    gi, gs = run_gpu(q, k, None, 64)
    ref = brute.kvstar_block_scores(q, k)
    assert np.allclose(gs, ref[gi], rtol=RTOL, atol=ATOL)
    kth = np.sort(ref)[::-1][63]
    assert np.all(ref[gi] >= kth - (ATOL + RTOL * kth))
    assert gs.sum() <= 8 * 32 * (1 + 1e-5)


def test_equal_scores_come_out_in_ascending_block_order():
    q, _ = make(14, 2, 4, 2, 16, 1, 1)
    k = np.full((8, 2, 2, 16), 0.25, np.float16)
    gi, gs = run_gpu(q, k, None, 3)
    assert gi.tolist() == [0, 1, 2]
    assert np.allclose(gs, 2 * 4 / 8, rtol=1e-6)


def test_module_api_like_the_reference_call_site():
    q, k = make(15, 3, 8, 2, 32, 50, 2)
    kvstar_retrieve.Setup(kvstar_retrieve.SetupParam(cpuNumaIds=[0], bindInfo=[(0, 0)],
                                                     deviceType=kvstar_retrieve.CPU,
                                                     totalTpSize=1, localRankId=0))
    tid = kvstar_retrieve.AsyncRetrieveByCPU(torch.from_numpy(q), torch.from_numpy(k), None, 6, 42,
                                             kvstar_retrieve.CPU)
    assert kvstar_retrieve.Wait(tid) == 0
    res = kvstar_retrieve.GetTaskResult(tid)
    assert res["status"] == "SUCCESS"
    oi, _, _ = c_api.kvstar_topk(q, k, 6)
    assert res["data"] == oi.tolist()
    assert kvstar_retrieve.Wait(tid) != 0          # the waiter is gone after the first Wait
    assert kvstar_retrieve.GetTaskResult(10 ** 9) is None
    # topK above the number of blocks returns every block
    tid = kvstar_retrieve.AsyncRetrieveByCPU(torch.from_numpy(q), torch.from_numpy(k), None, 80, 42,
                                             kvstar_retrieve.CPU)
    kvstar_retrieve.Wait(tid)
    assert sorted(kvstar_retrieve.GetTaskResult(tid)["data"]) == list(range(50))


def test_failures_are_reported_on_the_task():
    q, k = make(16, 2, 6, 4, 16, 10, 1)  # 6 q heads over 4 kv heads
    tid = kvstar_retrieve.AsyncRetrieveByCPU(torch.from_numpy(q), torch.from_numpy(k), None, 3, 1,
                                             kvstar_retrieve.CPU)
    assert kvstar_retrieve.Wait(tid) != 0
    res = kvstar_retrieve.GetTaskResult(tid)
    assert res["status"] == "FAILURE" and "divisible" in res["error"]
    q, k = make(17, 2, 4, 2, 16, 10, 1, d_orig=32)  # head dims differ and no pruning index
    tid = kvstar_retrieve.AsyncRetrieveByCPU(torch.from_numpy(q), torch.from_numpy(k), None, 3, 1,
                                             kvstar_retrieve.CPU)
    kvstar_retrieve.Wait(tid)
    assert "Dimension mismatch" in kvstar_retrieve.GetTaskResult(tid)["error"]
