"""CPU tests: the KVStar checker (oracle_kvstar_topk).

The reference's KVStar kernel cannot be compiled here (its translation unit includes the
project logger, which needs spdlog and fmt, neither of which the image has), and the reference
holds no test vectors for it.  The checker is therefore pinned by what the mathematics fixes:
closed forms, invariants and an independent float64 formulation built from library routines.
"""
import numpy as np
import pytest

from oracle import brute, c_api


def rand_case(seed, X=3, Hq=8, Hkv=2, d=32, n=24, M=4, scale=0.6):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((X, Hq, d)) * scale).astype(np.float16)
    k = (rng.standard_normal((n, M, Hkv, d)) * scale).astype(np.float16)
    return q, k


def test_matches_float64_formulation():
    for seed, kw in ((0, {}), (1, dict(X=1, Hq=4, Hkv=4, d=16, n=7, M=1)),
                     (2, dict(X=5, Hq=6, Hkv=3, d=20, n=40, M=3, scale=1.5))):
        q, k = rand_case(seed, **kw)
        idx, sc, allsc = c_api.kvstar_topk(q, k, 5)
        ref = brute.kvstar_block_scores(q, k)
        assert np.allclose(allsc, ref, rtol=1e-5, atol=1e-6)
        order = np.argsort(-ref, kind="stable")[:5]
        assert np.array_equal(idx, order)  # random data: no ties, the ranking is unambiguous
        assert np.array_equal(sc, allsc[idx])


def test_total_mass_is_one_per_query_row():
    # softmax rows sum to 1 -> the block scores sum to X * Hq whatever the inputs
    q, k = rand_case(3, X=4, Hq=8, Hkv=4)
    _, _, allsc = c_api.kvstar_topk(q, k, 1)
    assert allsc.sum() == pytest.approx(4 * 8, rel=1e-5)


def test_uniform_keys_give_equal_mass_and_the_heap_tie_order():
    # identical representatives -> every block holds M / S of each row's mass: X * Hq / n
    q, _ = rand_case(4, X=2, Hq=4, Hkv=2, d=16)
    k = np.broadcast_to(np.float16(0.25), (8, 2, 2, 16)).copy()
    idx, sc, allsc = c_api.kvstar_topk(q, k, 3)
    assert np.allclose(allsc, 2 * 4 / 8, rtol=1e-6)
    assert np.all(sc == allsc[0])
    # the reference's heap keeps (score, block) pairs and pops the smallest pair first: among
    # equal scores the larger block numbers stay, in descending order
    # (simd_compute_kernel.cpp:954-977); with eight equal blocks and topk 3 the first three fill
    # the heap and nothing replaces them
    assert idx.tolist() == [2, 1, 0]


def test_heap_tie_semantics_after_a_replacement():
    # two equal blocks then a better one, topk 2: the better block evicts the smaller pair
    # (block 0), leaving [2, 1].  zero queries make every score 0 -> equal mass per
    # representative, so mass is proportional to nothing but M; use keys to break it instead
    q = np.zeros((1, 1, 8), np.float16)
    q[0, 0, 0] = 1.0
    k = np.zeros((3, 1, 1, 8), np.float16)
    k[2, 0, 0, 0] = 2.0  # block 2 scores higher; blocks 0 and 1 tie exactly
    idx, sc, allsc = c_api.kvstar_topk(q, k, 2)
    assert allsc[0] == allsc[1] < allsc[2]
    assert idx.tolist() == [2, 1]
    e = np.exp(np.float64(2.0))
    assert np.allclose(allsc, np.array([1, 1, e]) / (2 + e), rtol=1e-6)  # closed form


def test_one_hot_limit():
    # one representative far above the rest takes all the mass of every row
    q = np.zeros((2, 2, 4), np.float16)
    q[..., 0] = 8.0
    k = np.zeros((5, 2, 1, 4), np.float16)
    k[3, 1, 0, 0] = 8.0  # score 64 against 0 elsewhere: exp(-64) vanishes in fp32 sums
    idx, sc, allsc = c_api.kvstar_topk(q, k, 1)
    assert idx.tolist() == [3] and sc[0] == pytest.approx(4.0, rel=1e-6)
    assert np.allclose(np.delete(allsc, 3), 0.0, atol=1e-20)


def test_channel_pruning_equals_slicing_the_queries():
    rng = np.random.default_rng(5)
    X, Hq, Hkv, d_orig, d = 2, 4, 2, 32, 12
    q = rng.standard_normal((X, Hq, d_orig)).astype(np.float16)
    k = rng.standard_normal((10, 2, Hkv, d)).astype(np.float16)
    pr = np.stack([rng.permutation(d_orig)[:d] for _ in range(Hkv)]).astype(np.int64)
    _, _, pruned = c_api.kvstar_topk(q, k, 4, pr)
    g = Hq // Hkv
    q_sliced = np.stack([q[:, H, pr[H // g]] for H in range(Hq)], axis=1)
    _, _, plain = c_api.kvstar_topk(q_sliced, k, 4)
    assert np.array_equal(pruned, plain)
    assert np.allclose(pruned, brute.kvstar_block_scores(q, k, pr), rtol=1e-5, atol=1e-6)


def test_gqa_head_mapping():
    # q head H reads kv head H // g: make kv head 1 the only informative one and check that only
    # the q heads of its group move the result
    rng = np.random.default_rng(6)
    q = rng.standard_normal((1, 4, 8)).astype(np.float16)
    k = np.zeros((6, 1, 2, 8), np.float16)
    k[:, :, 1] = rng.standard_normal((6, 1, 8)).astype(np.float16)
    _, _, base = c_api.kvstar_topk(q, k, 1)
    q2 = q.copy()
    q2[:, :2] = rng.standard_normal((1, 2, 8)).astype(np.float16)  # heads 0, 1 -> kv head 0 (zeros)
    _, _, same = c_api.kvstar_topk(q2, k, 1)
    assert np.array_equal(base, same)
    q3 = q.copy()
    q3[:, 2:] = -q[:, 2:]
    _, _, moved = c_api.kvstar_topk(q3, k, 1)
    assert not np.allclose(base, moved)


def test_fp16_conversion_table():
    # all 65536 half patterns (subnormals, infinities, NaNs) against numpy's conversion
    bits = np.arange(65536, dtype=np.uint16)
    got = c_api.half_to_float(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_topk_larger_than_blocks_and_count():
    q, k = rand_case(7, n=5)
    idx, sc, allsc = c_api.kvstar_topk(q, k, 9)
    assert idx.size == 5 and sorted(idx.tolist()) == list(range(5))
    assert np.all(np.diff(sc) <= 0)
