"""Pins the CPU oracle (oracle/ucm_oracle.c) before anything is compared against it.

Three independent anchors:
  1. golden outputs of the reference's own CPU backend (tests/golden/hash_retrieval_ref.npz,
     written by tests/golden/make_golden.py from hash_retrieval_backend.cpp);
  2. the numpy / pure-Python twin in oracle/brute.py (different formulation);
  3. closed forms and hand-made vectors.
"""
import os

import numpy as np
import pytest

import oracle
from oracle import brute, c_api
from helpers import (assert_topk_matches_unordered_ties, make_paged_case, random_codes, rng_for)

GOLD = os.path.join(os.path.dirname(__file__), "golden", "hash_retrieval_ref.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


# ----------------------------------------------------------------------------------------
# 1. golden vectors from the reference backend
# ----------------------------------------------------------------------------------------

def _c1_inputs():
    from golden.make_golden import c1_inputs, sha  # same generator as the fixture writer
    keys, q = c1_inputs()
    return keys, q, sha


def test_c1_inputs_reproduce(gold):
    keys, q, sha = _c1_inputs()
    assert sha(keys) == str(gold["c1_keys_sha256"])
    assert sha(q) == str(gold["c1_q_sha256"])


def test_c1_full_ranking_pins_every_block_score(gold):
    """k = 64 = every block: the reference's (index -> distance) map must equal the oracle's
    group-summed block-min distance for all 8 KV heads x 64 blocks."""
    keys, q, _ = _c1_inputs()
    table = np.arange(64, dtype=np.int32)[None, :]
    idx, dist = c_api.hamming_topk(q, keys, table, [8192], 64,
                                   flags=c_api.F_DISTANCE)  # ascending index order
    assert np.array_equal(idx[0], np.tile(np.arange(64), (8, 1)))
    for h in range(8):
        ref = np.zeros(64, np.int32)
        ref[gold["c1_idx64"][h]] = gold["c1_dist64"][h]
        assert np.array_equal(dist[0, h], ref)
        # the reference returns ascending distance
        assert np.all(np.diff(gold["c1_dist64"][h]) >= 0)


def test_c1_top16_matches_reference(gold):
    keys, q, _ = _c1_inputs()
    table = np.arange(64, dtype=np.int32)[None, :]
    idx, dist = c_api.hamming_topk(q, keys, table, [8192], 16,
                                   flags=c_api.F_DISTANCE | c_api.F_SCORE_ORDER)
    _, all_d = c_api.hamming_topk(q, keys, table, [8192], 64, flags=c_api.F_DISTANCE)
    for h in range(8):
        assert np.array_equal(dist[0, h], gold["c1_dist16"][h])  # same ascending distances
        assert_topk_matches_unordered_ties(idx[0, h], dist[0, h], gold["c1_idx16"][h],
                                           gold["c1_dist16"][h], all_scores=all_d[0, h])


def test_c1_similarity_is_full_minus_distance():
    keys, q, _ = _c1_inputs()
    table = np.arange(64, dtype=np.int32)[None, :]
    i1, s = c_api.hamming_topk(q, keys, table, [8192], 16)
    i2, d = c_api.hamming_topk(q, keys, table, [8192], 16, flags=c_api.F_DISTANCE)
    assert np.array_equal(i1, i2)
    assert np.array_equal(s, 4 * 128 - d)


@pytest.mark.parametrize("case,k", [("ragged", 5), ("ragged", 10), ("tail", 12), ("zero", 3)])
def test_backend_form_matches_reference(gold, case, k):
    data, query = gold[f"{case}_data"], gold[f"{case}_query"]
    if case == "ragged":
        indexes = gold["ragged_indexes"]
        ref_i, ref_d = gold[f"ragged_idx_k{k}"], gold[f"ragged_dist_k{k}"]
    else:
        n = data.shape[0]
        indexes = np.tile(np.arange(n, dtype=np.int32), (query.shape[0], 1))
        ref_i, ref_d = gold[f"{case}_idx"], gold[f"{case}_dist"]
    idx, dist, n = c_api.hash_retrieval(data, query, indexes, k)
    for r in range(query.shape[0]):
        kk = int(n[r])
        assert kk == int((ref_i[r] >= 0).sum())
        assert np.array_equal(dist[r, :kk], ref_d[r, :kk])
        # every block's true score, for the tie rule
        full_i, full_d, fn = c_api.hash_retrieval(data, query[r:r + 1], indexes[r:r + 1],
                                                  indexes.shape[1])
        score_of = {int(i): int(s) for i, s in zip(full_i[0, : fn[0]], full_d[0, : fn[0]])}
        assert_topk_matches_unordered_ties(idx[r, :kk], dist[r, :kk], ref_i[r, :kk],
                                           ref_d[r, :kk], all_scores=score_of)
        assert np.all(idx[r, kk:] == -1)


def test_zero_distance_block_found(gold):
    idx, dist, _ = c_api.hash_retrieval(gold["zero_data"], gold["zero_query"],
                                        np.arange(6, dtype=np.int32)[None, :], 3)
    assert idx[0, 0] == 3 and dist[0, 0] == 0


def test_ref_backend_loads_when_built():
    mod = oracle.ref_backend()
    if mod is None:
        pytest.skip("oracle/_ref not built in this environment")
    assert hasattr(mod, "HashRetrievalWorkerBackend")


# ----------------------------------------------------------------------------------------
# 2. C oracle vs the independent numpy twin
# ----------------------------------------------------------------------------------------

@pytest.mark.parametrize("seed,B,Hq,Hkv,Wd,BS,lens,k,sink,recent", [
    (11, 2, 8, 2, 4, 16, [100, 37], 3, 0, 0),
    (12, 3, 4, 4, 2, 8, [64, 1, 23], 4, 0, 0),
    (13, 2, 8, 1, 8, 16, [90, 160], 5, 0, 0),       # MLA-like: one KV head, 8 q heads
    (14, 2, 8, 2, 4, 16, [100, 75], 4, 16, 32),     # sink + recent
    (15, 1, 6, 3, 3, 4, [19], 2, 3, 1),             # odd sizes, W not a multiple of 4
    (16, 2, 4, 2, 4, 16, [0, 48], 2, 0, 0),         # an empty request
    (17, 1, 4, 2, 4, 16, [40], 8, 0, 0),            # k larger than the block count
])
@pytest.mark.parametrize("reduce_heads", [False, True])
def test_topk_matches_brute(seed, B, Hq, Hkv, Wd, BS, lens, k, sink, recent, reduce_heads):
    q, kc, table, lens = make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens, table_pad=2)
    for physical in (False, True):
        for score_order in (False, True):
            for distance in (False, True):
                flags = ((c_api.F_REDUCE_HEADS if reduce_heads else 0)
                         | (c_api.F_PHYSICAL if physical else 0)
                         | (c_api.F_SCORE_ORDER if score_order else 0)
                         | (c_api.F_DISTANCE if distance else 0))
                i1, s1 = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags)
                i2, s2 = brute.hamming_topk(q, kc, table, lens, k, sink, recent, reduce_heads,
                                            physical, score_order, distance)
                assert np.array_equal(i1, i2)
                assert np.array_equal(s1, s2)


def test_head_major_layout_is_the_same_function():
    q, kc, table, lens = make_paged_case(21, 2, 8, 4, 4, 16, [70, 33])
    i1, s1 = c_api.hamming_topk(q, kc, table, lens, 3)
    kc_hm = np.ascontiguousarray(kc.transpose(0, 2, 1, 3))
    i2, s2 = c_api.hamming_topk(q, kc_hm, table, lens, 3, head_major=True)
    assert np.array_equal(i1, i2) and np.array_equal(s1, s2)


def test_threads_do_not_change_results():
    q, kc, table, lens = make_paged_case(22, 5, 8, 2, 4, 16, [70, 33, 160, 16, 5])
    a = c_api.hamming_topk(q, kc, table, lens, 4, nthreads=1)
    b = c_api.hamming_topk(q, kc, table, lens, 4, nthreads=5)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_per_token_scores_vs_block_scores():
    """Block min of the per-token output (hamming_topk.py:45-47) == G*bits - block score."""
    q, kc, table, lens = make_paged_case(23, 2, 8, 2, 4, 16, [100, 48], table_pad=1)
    BS, max_blocks = 16, table.shape[1]
    for sink, recent in ((0, 0), (16, 32), (5, 3)):
        tok = c_api.hamming_score(q, kc, table, lens, max_blocks * BS, sink, recent)
        blk = tok.reshape(2, 2, max_blocks, BS).min(axis=-1)
        bs = brute.block_scores(q, kc, table, lens, sink, recent)
        for b in range(2):
            n = bs[b].shape[1]
            assert np.array_equal(4 * 128 - blk[b, :, :n], bs[b])
            assert np.all(blk[b, :, n:] == c_api.INF)
        red = c_api.hamming_score(q, kc, table, lens, max_blocks * BS, sink, recent,
                                  reduce_heads=True)
        assert np.array_equal(red[:, 0], tok.min(axis=1))


# ----------------------------------------------------------------------------------------
# 3. closed forms and hand-made vectors
# ----------------------------------------------------------------------------------------

def test_identical_and_complement_codes():
    rng = rng_for(31)
    kc = random_codes(rng, (4, 8, 2, 4))
    table = np.arange(4, dtype=np.int32)[None, :]
    # all 4 query heads of KV head 0 equal token (2,5) of head 0 -> block 2 scores G*bits
    q = np.zeros((1, 8, 4), np.uint32)
    q[0, 0:4] = kc[2, 5, 0]
    q[0, 4:8] = ~kc[1, 3, 1]  # complement of a head-1 token: that token contributes 0
    idx, s = c_api.hamming_topk(q, kc, table, [32], 1)
    assert idx[0, 0, 0] == 2 and s[0, 0, 0] == 4 * 128
    tok = c_api.hamming_score(q, kc, table, [32], 32)
    assert tok[0, 0, 2 * 8 + 5] == 0
    assert tok[0, 1, 1 * 8 + 3] == 4 * 128


def test_all_equal_scores_select_lowest_indices():
    kc = np.zeros((10, 4, 1, 4), np.uint32)
    q = np.zeros((1, 2, 4), np.uint32)
    table = np.arange(10, dtype=np.int32)[::-1][None, :].copy()
    idx, s = c_api.hamming_topk(q, kc, table, [40], 4)
    assert idx[0, 0].tolist() == [0, 1, 2, 3]
    assert np.all(s == 2 * 128)
    idx, _ = c_api.hamming_topk(q, kc, table, [40], 4, flags=c_api.F_PHYSICAL)
    assert idx[0, 0].tolist() == [9, 8, 7, 6]


def test_single_bit_distance_by_hand():
    kc = np.zeros((1, 2, 1, 1), np.uint32)
    kc[0, 0, 0, 0] = 0b1011
    kc[0, 1, 0, 0] = 0b0001
    q = np.array([[[0b0001], [0b0011]]], np.uint32)  # G = 2
    tok = c_api.hamming_score(q, kc, np.zeros((1, 1), np.int32), [2], 2)
    # token0: popc(1011^0001)=2, popc(1011^0011)=1 -> 3 ; token1: 0 + 1 -> 1
    assert tok[0, 0].tolist() == [3, 1]
    idx, s = c_api.hamming_topk(q, kc, np.zeros((1, 1), np.int32), [2], 1)
    assert s[0, 0, 0] == 2 * 32 - 1


def test_garbage_past_seq_len_is_masked():
    q, kc, table, lens = make_paged_case(33, 1, 4, 2, 4, 16, [37])
    a = c_api.hamming_topk(q, kc, table, lens, 2)
    kc2 = kc.copy()
    pb = table[0, 2]
    kc2[pb, 37 - 32:] = q[0, 0]  # would be a perfect match if it were read
    b = c_api.hamming_topk(q, kc2, table, lens, 2)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_out_of_range_table_entry_scores_minus_one():
    q, kc, table, lens = make_paged_case(34, 1, 4, 2, 4, 16, [48])
    table[0, 1] = kc.shape[0] + 5
    idx, s = c_api.hamming_topk(q, kc, table, lens, 3)
    assert s[0, 0, 1] == -1 and idx[0, 0].tolist() == [0, 1, 2]


def test_update_seq_lens_values():
    # hamming_topk.py:7-12 by hand: len 1000, topk 256, BS 128 -> over 744 -> 6 blocks dropped
    out = c_api.update_seq_lens([1000, 256, 100, 257, 0], 256, 128)
    assert out.tolist() == [1000 - 6 * 128, 256, 100, 257 - 128, 0]
    assert np.array_equal(out, brute.update_seq_lens([1000, 256, 100, 257, 0], 256, 128))


def test_encoder_bit_and_byte_order():
    K = N = 64
    W = np.eye(K, dtype=np.float32)
    x = np.zeros((3, K), np.float32)
    x[0, 0] = 1.0    # bit 0 of word 0
    x[1, 9] = 2.0    # byte 1 bit 1
    x[2, 37] = 0.5   # word 1 bit 5
    x[2, 3] = -1.0   # negative -> 0
    c = c_api.hash_encode(x, W)
    assert c.tolist() == [[1, 0], [1 << 9, 0], [0, 1 << 5]]
    assert c.view(np.uint8)[1].tolist()[:2] == [0, 2]
    assert np.array_equal(c, brute.hash_encode(x, W))


def test_encoder_zero_and_nan_give_zero_bit():
    W = np.eye(32, dtype=np.float32)
    x = np.zeros((2, 32), np.float32)
    x[0, 1] = -0.0
    x[0, 3] = 1e-30
    x[1, 2] = np.nan   # NaN * 0 = NaN: every projection of the row is NaN -> all bits 0
    x[1, 5] = 1.0
    c = c_api.hash_encode(x, W)
    assert c[0, 0] == 0b1000
    assert c[1, 0] == 0


def test_encoder_negation_gives_complement_and_margin_rule():
    rng = rng_for(41)
    x = rng.standard_normal((64, 128)).astype(np.float32)
    W = rng.standard_normal((128, 128)).astype(np.float32)
    c32, margin = c_api.hash_encode(x, W, want_margin=True)
    c64 = c_api.hash_encode(x, W, acc_f64=True)
    cb = brute.hash_encode(x, W)
    assert np.array_equal(c64, cb)
    diff = brute.unpack_pm(c32) != brute.unpack_pm(cb)
    assert not np.any(diff & (margin >= 1e-2))  # fp32 vs fp64 may flip only tiny margins
    assert np.allclose(margin, brute.margins(x, W), rtol=1e-4, atol=1e-6)
    cneg = c_api.hash_encode(-x, W)
    assert np.array_equal(cneg, ~c32)  # no projection is exactly 0 for Gaussian data


def test_encode_cache_and_scatter():
    rng = rng_for(42)
    T, H, K, N, NB, BS = 9, 2, 32, 64, 4, 4
    x = rng.standard_normal((T, H, K)).astype(np.float32)
    W = rng.standard_normal((2, K, N)).astype(np.float32)
    slot = np.array([0, 5, 15, -1, 16, 7, 3, 100, 9], np.int64)  # -1, 16, 100 are skipped
    cache = np.full((NB, BS, H, N // 32), 0xDEADBEEF, np.uint32)
    c_api.hash_encode_cache(x, W, 1, slot, cache, BS)
    codes = np.stack([c_api.hash_encode(x[:, h], W[h]) for h in range(H)], axis=1)
    expect = np.full_like(cache, 0xDEADBEEF)
    for t, s in enumerate(slot):
        if 0 <= s < NB * BS:
            expect[s // BS, s % BS] = codes[t]
    assert np.array_equal(cache, expect)
    cache2 = np.full_like(cache, 0xDEADBEEF)
    c_api.code_scatter(codes, slot, cache2, BS)
    assert np.array_equal(cache2, expect)


def test_encode_paged_is_gather_plus_prefix_slot_mapping():
    """The rehash of keys that sit in the paged KV cache must equal the reference's recipe
    written out with numpy: gather the blocks, keep the first n tokens, slot(i) =
    block_ids[i // BS] * BS + i % BS (gsa_on_device.py:574-588, :1142-1174).  The slot rule is
    also checked by hand on one token."""
    rng = rng_for(44)
    NBk, NB, BS, H, K, N = 7, 6, 4, 2, 32, 64
    kc = rng.standard_normal((NBk, BS, H, K)).astype(np.float32)
    W = rng.standard_normal((1, K, N)).astype(np.float32)
    ids = np.array([5, 2, 6, 0], np.int32)  # 6 exists in the KV cache but not in the code cache
    n_tokens = 14                          # the last block is half used
    cache = np.full((NB, BS, H, N // 32), 0xDEADBEEF, np.uint32)
    c_api.hash_encode_paged(kc, ids, n_tokens, W, 0, cache)
    gathered = kc[np.clip(ids, 0, NBk - 1)].reshape(-1, H, K)[:n_tokens]
    token_idx = np.arange(n_tokens)
    slots = ids[token_idx // BS].astype(np.int64) * BS + token_idx % BS
    slots[ids[token_idx // BS] >= NB] = -1
    expect = np.full_like(cache, 0xDEADBEEF)
    c_api.hash_encode_cache(gathered, W, 0, slots, expect, BS)
    assert np.array_equal(cache, expect)
    # token 5 = token 1 of block ids[1] = 2 -> slot 9
    assert np.array_equal(cache[2, 1, 0], c_api.hash_encode(kc[2, 1, :1], W[0])[0])
    assert (cache[0, 2:] == 0xDEADBEEF).all()  # tokens 14, 15 of the last block were not encoded
    assert (cache[[1, 3, 4]] == 0xDEADBEEF).all()


def test_gather_scatter_roundtrip_and_addresses():
    rng = rng_for(43)
    size, n = 48, 7
    pool = rng.integers(0, 256, size=(20, size), dtype=np.uint8)
    ids = rng.permutation(20)[:n]
    flat = c_api.gather([pool[i] for i in ids], size)
    assert np.array_equal(flat.reshape(n, size), pool[ids])
    dst = np.zeros_like(pool)
    ids2 = rng.permutation(20)[:n]
    c_api.scatter(flat, [dst[i] for i in ids2], size)
    assert np.array_equal(dst[ids2], pool[ids])
    untouched = np.setdiff1d(np.arange(20), ids2)
    assert not dst[untouched].any()
    # address rule by hand: base + id * bytes
    a = c_api.block_addrs([1000, 2000], [16, 32], [3, 0])
    assert a.tolist() == [[1048, 2096], [1000, 2000]]


def test_paged_copy_variable_columns():
    rng = rng_for(44)
    col_bytes = [32, 16, 48]
    nb = 6
    cols = [rng.integers(0, 256, size=(nb, cb), dtype=np.uint8) for cb in col_bytes]
    base = [c.ctypes.data for c in cols]
    ids = np.array([4, 1, 5], np.int32)
    flat = np.zeros(len(ids) * sum(col_bytes), np.uint8)
    c_api.paged_copy(base, col_bytes, ids, flat, to_cache=False)
    expect = np.concatenate([np.concatenate([c[i] for c in cols]) for i in ids])
    assert np.array_equal(flat, expect)
    cols2 = [np.zeros_like(c) for c in cols]
    ids2 = np.array([0, 2, 3], np.int32)
    c_api.paged_copy([c.ctypes.data for c in cols2], col_bytes, ids2, flat, to_cache=True)
    for c, c2 in zip(cols, cols2):
        assert np.array_equal(c2[ids2], c[ids])


def test_topk_request_head_items_mode_equals_the_request_mode():
    """The timing variant that hands (request, KV head) items to pinned threads computes the
    same lists as one thread per request."""
    q, kc, table, lens = make_paged_case(4711, 3, 8, 4, 2, 8, [70, 33, 8], table_pad=1)
    ref = c_api.hamming_topk(q, kc, table, lens, 3, 4, 8)
    for nt in (1, 2, 5):
        got = c_api.hamming_topk(q, kc, table, lens, 3, 4, 8, nthreads=nt, head_items=True)
        assert np.array_equal(got[0], ref[0]) and np.array_equal(got[1], ref[1])
