"""GPU parity of the float retrieval path (ucm_dot_topk) against the CPU checker, the golden
outputs of the reference's ESA backend and exact float64 scores.

Tolerance (floating point): a score may differ from the sequential-fp32 reference by at most
TOL_REL * sum_d |q_d * x_d| (the fp32 partial sums are added in another order); indices may
differ from the reference's only between candidates whose exact scores are closer than that.
Integer-valued inputs, whose sums are exact in fp32, must match bit for bit.
"""
import os

import numpy as np
import pytest
import torch

from golden.make_golden_esa import dense_inputs, wide_inputs
from helpers import rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu

TOL_REL = 1e-5
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "esa_retrieval_ref.npz"))


def gpu_dot_topk(data, query, indexes, k):
    from ucm_amd.sparse.esa_retrieval_worker import dot_topk

    i, s = dot_topk(torch.from_numpy(data).cuda(), torch.from_numpy(query).cuda(),
                    torch.from_numpy(indexes).cuda(), k)
    return i.cpu().numpy(), s.cpu().numpy()


def check(data, query, indexes, k, ref=None):
    gi, gs = gpu_dot_topk(data, query, indexes, k)
    oi, osc = ref if ref is not None else c_api.dot_topk(data, query, indexes, k)
    d64, q64 = data.astype(np.float64), query.astype(np.float64)
    for b in range(query.shape[0]):
        valid = [(j, int(i)) for j, i in enumerate(indexes[b]) if 0 <= i < data.shape[0]]
        kk = min(k, len(valid))
        exact = {i: float(q64[b] @ d64[i]) for _, i in valid}
        mag = {i: float(np.abs(q64[b] * d64[i]).sum()) for _, i in valid}
        tol = TOL_REL * max(mag.values(), default=0.0)
        assert (gi[b, kk:] == -1).all() and (gs[b, kk:] == 0).all()
        assert (oi[b, kk:] == -1).all()
        sel = gi[b, :kk].tolist()
        pos_of = {}
        for j, i in valid:
            pos_of.setdefault(i, j)
        # every selected candidate is allowed; no list position is used twice
        assert all(i in exact for i in sel)
        if len({i for _, i in valid}) == len(valid):
            assert len(set(sel)) == kk
        # scores: close to exact, descending, and position by position close to the reference
        for t in range(kk):
            assert abs(gs[b, t] - exact[sel[t]]) <= tol
            assert abs(gs[b, t] - osc[b, t]) <= 2 * tol
            if t:
                assert gs[b, t - 1] >= gs[b, t]
        # set: nothing clearly better than the k-th was left out
        if kk:
            kth = sorted(exact.values(), reverse=True)[kk - 1]
            assert all(exact[i] >= kth - 2 * tol for i in sel)
            assert all(i in sel for i in exact if exact[i] > kth + 2 * tol)
        # indices equal the reference's except between near-ties
        for t in range(kk):
            if gi[b, t] != oi[b, t]:
                assert abs(exact[int(gi[b, t])] - exact[int(oi[b, t])]) <= 2 * tol
    return gi, gs


def test_golden_cases_of_the_reference_backend():
    data, query, indexes = dense_inputs()
    check(data, query, indexes, 16, ref=(GOLD["dense_idx"], GOLD["dense_score"]))
    data, query, indexes = wide_inputs()
    check(data, query, indexes, 100, ref=(GOLD["wide_idx"], GOLD["wide_score"]))
    check(GOLD["ragged_data"], GOLD["ragged_query"], GOLD["ragged_indexes"], 5,
          ref=(GOLD["ragged_idx"], GOLD["ragged_score"]))


def test_integer_inputs_are_bit_exact_and_ties_keep_list_order():
    data, query = GOLD["ints_data"], GOLD["ints_query"]
    indexes = np.tile(np.arange(50, dtype=np.int32), (2, 1))
    gi, gs = gpu_dot_topk(data, query, indexes, 50)
    oi, osc = c_api.dot_topk(data, query, indexes, 50)
    assert np.array_equal(gs, GOLD["ints_score"])  # the reference's scores, exactly
    assert np.array_equal(gi, oi) and np.array_equal(gs, osc)


@pytest.mark.parametrize("n_items,dim,B,max_n,k", [
    (5000, 1024, 2, 3000, 1000),     # the reference driver's shape, scaled (retrieval_worker.py:45-60)
    (300, 128, 5, 300, 300),         # k = every candidate: a full sort
    (1000, 100, 3, 257, 64),         # dim % 4 == 0 but not a multiple of 256
    (400, 30, 4, 77, 10),            # dim % 4 != 0: scalar loads
    (64, 4096, 1, 64, 7),            # long rows
    (20000, 64, 8, 6000, 4096),      # the largest k
    (30000, 32, 2, 10000, 500),      # more than 8192 candidates: keys re-read from memory per phase
    (9000, 16, 2, 8192, 100),        # exactly what the register path holds
    (9000, 16, 2, 8193, 100),        # one more
    (2000, 16, 3, 1024, 40),         # the longest row of the counting path
    (2000, 16, 3, 1025, 40),         # the shortest row of the search-and-sort path
])
def test_random_shapes(n_items, dim, B, max_n, k):
    rng = rng_for(n_items + dim + B)
    data = rng.standard_normal((n_items, dim)).astype(np.float32)
    query = rng.standard_normal((B, dim)).astype(np.float32)
    indexes = np.stack([rng.permutation(n_items)[:max_n] if max_n <= n_items
                        else rng.integers(0, n_items, max_n) for _ in range(B)]).astype(np.int32)
    # ragged tails, holes and entries outside the matrix
    if B > 1:
        indexes[1, max_n // 2:] = -1
        indexes[-1, ::7] = -1
        indexes[0, 3] = n_items + 5
    check(data, query, indexes, k)


@pytest.mark.parametrize("max_n,k,values", [
    (5000, 2000, 9),      # nine distinct scores: every bucket of the ordering fast path overflows
    (8000, 3000, 1),      # all scores equal: the output is the list order
    (3000, 2500, 400),    # a few hundred distinct scores: crowded and sparse buckets mixed
    (20000, 4096, 30),    # the same past the register-resident size
])
def test_many_equal_scores_are_bit_exact_in_list_order(max_n, k, values):
    """Integer-valued data make the scores exact in any summation order, so outputs must equal
    the checker's bit for bit, including the order among equal scores (list order)."""
    rng = rng_for(max_n + values)
    n_items, dim = 25000, 8
    data = rng.integers(0, 2, size=(n_items, dim)).astype(np.float32)
    if values == 1:
        data[:] = 1.0
    elif values > 9:
        data[:, 0] = rng.integers(0, values, n_items)
    query = np.ones((2, dim), np.float32)
    indexes = np.stack([rng.permutation(n_items)[:max_n] for _ in range(2)]).astype(np.int32)
    gi, gs = gpu_dot_topk(data, query, indexes, k)
    oi, osc = c_api.dot_topk(data, query, indexes, k)
    assert np.array_equal(gs, osc)
    # equal scores: the checker's order among ties is its partial_sort's; list order is this
    # library's contract, so compare against a stable sort of the exact scores
    exact = (data[indexes] * query[:, None, :]).sum(-1)
    for b in range(2):
        order = np.argsort(-exact[b], kind="stable")[:k]
        assert np.array_equal(gi[b], indexes[b][order])


def test_fewer_candidates_than_k_and_empty_rows():
    rng = rng_for(9)
    data = rng.standard_normal((100, 64)).astype(np.float32)
    query = rng.standard_normal((3, 64)).astype(np.float32)
    indexes = -np.ones((3, 40), np.int32)
    indexes[0, :40] = rng.permutation(100)[:40]
    indexes[1, 5:9] = [3, 99, 0, 50]
    gi, gs = check(data, query, indexes, 16)
    assert (gi[2] == -1).all() and (gs[2] == 0).all()
    assert (gi[1, 4:] == -1).all() and sorted(gi[1, :4].tolist()) == [0, 3, 50, 99]


def test_nan_and_inf_scores_sort_below_and_above_numbers():
    data = np.ones((6, 8), np.float32)
    data[1, 0] = np.nan
    data[2, 0] = np.inf
    data[3, 0] = -np.inf
    data[4] *= 2
    query = np.ones((1, 8), np.float32)
    indexes = np.arange(6, dtype=np.int32)[None, :]
    gi, gs = gpu_dot_topk(data, query, indexes, 6)
    assert gi[0].tolist() == [2, 4, 0, 5, 3, 1]
    assert gs[0, 0] == np.inf and gs[0, 4] == -np.inf and np.isnan(gs[0, 5])


def test_worker_api_matches_the_reference_backend_outputs():
    from ucm_amd.sparse.esa_retrieval_worker import RetrievalWorker, RetrievalWorkerBackend

    data, query, indexes = dense_inputs()
    w = RetrievalWorker(RetrievalWorkerBackend(data, {0: [0]}))
    rid = w.submit(torch.from_numpy(query).to(torch.float64), 16, indexes)  # handle_input converts
    assert isinstance(w.poll(rid), bool)
    w.wait(rid)
    r = w.get_result(rid)
    assert r["indices"].shape == (2, 16)
    assert np.array_equal(r["indices"], GOLD["dense_idx"])  # no near-ties in this case
    assert np.allclose(r["scores"], GOLD["dense_score"], rtol=0, atol=1e-4)
    with pytest.raises(RuntimeError):
        w.get_result(rid)                       # consumed once
    with pytest.raises(RuntimeError):
        w.wait(12345)
    with pytest.raises(RuntimeError):
        w.submit(torch.zeros(2, 64), 4, indexes)
    with pytest.raises(RuntimeError):
        w.submit(torch.from_numpy(query), 4, indexes[:1])


def test_argument_errors():
    from ucm_amd.sparse.esa_retrieval_worker import dot_topk

    d = torch.zeros((10, 8), device="cuda")
    q = torch.zeros((2, 8), device="cuda")
    i = torch.zeros((2, 4), dtype=torch.int32, device="cuda")
    with pytest.raises(NotImplementedError):
        dot_topk(d, q, i, 5000)
    with pytest.raises(ValueError):
        dot_topk(d, q, i, 0)
    with pytest.raises(ValueError):
        dot_topk(d.cpu(), q, i, 2)
    with pytest.raises(ValueError):
        dot_topk(d, q, i.long(), 2)
    oi, osc = dot_topk(d, q[:0], i[:0], 3)
    assert oi.shape == (0, 3)
