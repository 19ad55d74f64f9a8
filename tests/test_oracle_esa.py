"""CPU tests: the float-retrieval checker (oracle_dot_topk) against outputs of the reference's
own ESA backend (tests/golden/esa_retrieval_ref.npz, written by make_golden_esa.py)."""
import os

import numpy as np

from golden.make_golden_esa import dense_inputs, wide_inputs
from oracle import c_api

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "esa_retrieval_ref.npz"))


def assert_same_ranking(idx, sc, ref_idx, ref_sc, exact64, tol):
    """Ranking equality up to ties: identical scores position by position (within tol), and
    where the indices differ the two candidates' exact scores differ by less than tol."""
    assert idx.shape == ref_idx.shape
    assert np.allclose(sc, ref_sc, rtol=0, atol=tol)
    for b in range(idx.shape[0]):
        for t in np.nonzero(idx[b] != ref_idx[b])[0]:
            assert idx[b, t] >= 0 and ref_idx[b, t] >= 0
            assert abs(exact64[b][idx[b, t]] - exact64[b][ref_idx[b, t]]) <= tol


def exact(data, query):
    return query.astype(np.float64) @ data.astype(np.float64).T  # [B, n_items]


def test_dense_and_wide_match_the_reference_backend_bit_for_bit():
    # same sequential fp32 arithmetic -> the scores are identical, not merely close
    for inputs, name, k in ((dense_inputs, "dense", 16), (wide_inputs, "wide", 100)):
        data, query, indexes = inputs()
        assert np.array_equal(indexes, GOLD[f"{name}_indexes"])
        oi, osc = c_api.dot_topk(data, query, indexes, k)
        assert np.array_equal(osc, GOLD[f"{name}_score"])
        assert_same_ranking(oi, osc, GOLD[f"{name}_idx"], GOLD[f"{name}_score"], exact(data, query), 0.0)


def test_ragged_lists_and_padding():
    data, query, indexes = GOLD["ragged_data"], GOLD["ragged_query"], GOLD["ragged_indexes"]
    oi, osc = c_api.dot_topk(data, query, indexes, 5)
    assert np.array_equal(oi, GOLD["ragged_idx"])
    assert np.array_equal(osc, GOLD["ragged_score"])
    assert oi[1].tolist()[3:] == [-1, -1] and osc[1].tolist()[3:] == [0.0, 0.0]  # 3 candidates, k = 5


def test_exact_integer_scores_and_ties():
    data, query = GOLD["ints_data"], GOLD["ints_query"]
    indexes = np.tile(np.arange(50, dtype=np.int32), (2, 1))
    oi, osc = c_api.dot_topk(data, query, indexes, 50)
    assert np.array_equal(osc, GOLD["ints_score"])          # exact arithmetic: no freedom at all
    assert np.array_equal(osc, np.sort(exact(data, query), axis=1)[:, ::-1].astype(np.float32))
    ex = exact(data, query)
    for b in range(2):
        assert sorted(oi[b].tolist()) == list(range(50))
        assert np.array_equal(ex[b][oi[b]], ex[b][GOLD["ints_idx"][b]])
        # equal scores keep list order (rows 7 and 21 are identical; small integers tie often)
        for t in range(49):
            if osc[b, t] == osc[b, t + 1]:
                assert oi[b, t] < oi[b, t + 1]
        assert oi[b].tolist().index(7) < oi[b].tolist().index(21)


def test_descending_order_closed_form_and_out_of_range_entries():
    # data = one-hot rows scaled by their index: dot(q, row_i) = i * q[i % dim]
    dim, n = 8, 24
    data = np.zeros((n, dim), np.float32)
    for i in range(n):
        data[i, i % dim] = i
    query = np.ones((1, dim), np.float32)
    indexes = np.array([[5, -1, 23, 100, 2, 17, -7, 9]], np.int32)  # 100 and -7 are no candidates
    oi, osc = c_api.dot_topk(data, query, indexes, 4)
    assert oi.tolist() == [[23, 17, 9, 5]] and osc.tolist() == [[23.0, 17.0, 9.0, 5.0]]
    oi, osc = c_api.dot_topk(data, query, indexes, 8)
    assert oi.tolist() == [[23, 17, 9, 5, 2, -1, -1, -1]]
