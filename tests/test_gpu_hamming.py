"""GPU parity: the HIP Hamming scorer / block top-k against the CPU oracle, bit-exact.

Every call goes through the C ABI (ctypes) via the host-side mirror in ucm_amd.sparse.
"""
import os

import numpy as np
import pytest
import torch

from helpers import half_piece_sums, make_paged_case, random_codes, rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "hash_retrieval_ref.npz")


def dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.cuda()


def as_i32(a):
    return np.ascontiguousarray(a).view(np.int32)


def run_gpu(q, kc, table, lens, k, sink=0, recent=0, head_major=False, **kw):
    from ucm_amd.sparse import hamming_topk

    kc_in = np.ascontiguousarray(kc.transpose(0, 2, 1, 3)) if head_major else kc
    idx, sc = hamming_topk(dev(as_i32(q)), dev(as_i32(kc_in)),
                           dev(table) if table is not None else None, dev(lens), k, sink, recent,
                           head_major=head_major, **kw)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), sc.cpu().numpy()


def run_oracle(q, kc, table, lens, k, sink=0, recent=0, reduce_heads=False,
               return_physical=False, score_order=False, distance=False, max_blocks=None):
    flags = ((c_api.F_REDUCE_HEADS if reduce_heads else 0)
             | (c_api.F_PHYSICAL if return_physical else 0)
             | (c_api.F_SCORE_ORDER if score_order else 0)
             | (c_api.F_DISTANCE if distance else 0))
    return c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=max_blocks)


def check(q, kc, table, lens, k, sink=0, recent=0, head_major=False, **kw):
    oi, os_ = run_oracle(q, kc, table, lens, k, sink, recent, **kw)
    for _ in range(2):  # twice: a call must not depend on what the previous one left behind
        gi, gs = run_gpu(q, kc, table, lens, k, sink, recent, head_major, **kw)
        assert np.array_equal(gi, oi), (gi, oi)
        assert np.array_equal(gs, os_), (gs, os_)


def test_config1_golden_and_oracle():
    """BASELINE.json config 1 against the reference CPU backend's recorded output."""
    from golden.make_golden import c1_inputs

    gold = np.load(GOLD)
    keys, q = c1_inputs()
    table = np.arange(64, dtype=np.int32)[None, :]
    lens = np.array([8192], np.int32)
    check(q, keys, table, lens, 16)
    # every block's distance, by index, equals what the reference computed
    gi, gd = run_gpu(q, keys, table, lens, 64, distance=True)
    for h in range(8):
        ref = np.zeros(64, np.int32)
        ref[gold["c1_idx64"][h]] = gold["c1_dist64"][h]
        assert np.array_equal(gd[0, h], ref)
    # score-ordered top-16 distances are the reference's ascending distances
    gi, gd = run_gpu(q, keys, table, lens, 16, distance=True, score_order=True)
    for h in range(8):
        assert np.array_equal(gd[0, h], gold["c1_dist16"][h])


# (seed, B, Hq, Hkv, Wd, BS, lens, k) — fast path: Wd in {4,8,16}, contiguous token-major
FAST_CASES = [
    (101, 2, 32, 8, 4, 128, [1000, 4096], 8),       # the Llama-3 layout, G=4
    (102, 3, 8, 8, 4, 128, [128, 129, 1], 2),        # G=1
    (103, 2, 16, 8, 4, 64, [700, 64], 4),            # G=2
    (104, 2, 64, 8, 4, 128, [2000, 900], 5),         # G=8  -> 4 bit planes
    (105, 2, 128, 1, 8, 64, [3000, 640], 16),        # MLA-like: G=128, 256-bit codes
    (106, 1, 24, 2, 16, 32, [999], 7),               # G=12, 512-bit codes
    (107, 2, 40, 4, 4, 16, [100, 333], 6),           # G=10, small blocks (several per workgroup)
    (108, 1, 3, 1, 4, 64, [500], 3),                 # G=3 (planes), one KV head
    (109, 2, 32, 16, 4, 128, [300, 5000], 9),        # 16 KV heads
    (110, 4, 32, 8, 4, 128, [0, 128, 127, 16384], 64),  # empty request, k > nblk, long
    (111, 2, 32, 8, 4, 128, [131072, 100000], 128),  # 1024 blocks per request
    (112, 2, 128, 1, 8, 64, [65536, 30000], 128),    # config 5 shape at 2 requests
    (113, 2, 16, 4, 4, 48, [1000, 48], 5),           # 3 KiB blocks: several whole blocks per wave
    (114, 1, 64, 32, 4, 128, [2000], 6),             # 32 KV heads: 64 KiB blocks split over waves
    (115, 2, 20, 4, 8, 16, [700, 50], 4),            # 2 KiB blocks, G=5, 256-bit codes, 4 heads
]


@pytest.mark.parametrize("seed,B,Hq,Hkv,Wd,BS,lens,k", FAST_CASES)
def test_fast_path_matches_oracle(seed, B, Hq, Hkv, Wd, BS, lens, k):
    q, kc, table, lens = make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens, table_pad=3)
    check(q, kc, table, lens, k)
    check(q, kc, table, lens, k, reduce_heads=True)
    check(q, kc, table, lens, k, return_physical=True, distance=True)
    check(q, kc, table, lens, k, score_order=True)


GENERIC_CASES = [
    (201, 2, 6, 3, 3, 4, [19, 7], 2),       # odd everything
    (202, 1, 8, 2, 18, 16, [100], 3),       # 576-bit codes (18 words), the MLA nope+rope width
    (203, 2, 8, 4, 2, 8, [64, 30], 4),      # 64-bit codes
    (204, 1, 4, 1, 4, 8, [40], 2),          # block too small for the fast path
]


@pytest.mark.parametrize("seed,B,Hq,Hkv,Wd,BS,lens,k", GENERIC_CASES)
def test_generic_path_matches_oracle(seed, B, Hq, Hkv, Wd, BS, lens, k):
    q, kc, table, lens = make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens, table_pad=1)
    check(q, kc, table, lens, k)
    check(q, kc, table, lens, k, reduce_heads=True, score_order=True)


def test_head_major_cache_layout():
    q, kc, table, lens = make_paged_case(301, 2, 32, 8, 4, 128, [700, 1500])
    check(q, kc, table, lens, 4, head_major=True)


@pytest.mark.parametrize("sink,recent", [(128, 512), (1, 1), (200, 0), (0, 300)])
def test_sink_and_recent(sink, recent):
    q, kc, table, lens = make_paged_case(302, 3, 32, 8, 4, 128, [5000, 640, 100], table_pad=2)
    check(q, kc, table, lens, 12, sink, recent)
    check(q, kc, table, lens, 12, sink, recent, reduce_heads=True, return_physical=True)


def test_ties_go_to_lower_index():
    kc = np.zeros((40, 64, 8, 4), np.uint32)
    q = np.zeros((1, 32, 4), np.uint32)
    table = np.arange(40, dtype=np.int32)[::-1][None, :].copy()
    gi, gs = run_gpu(q, kc, table, np.array([40 * 64], np.int32), 5)
    assert np.array_equal(gi[0], np.tile(np.arange(5), (8, 1)))
    assert np.all(gs == 4 * 128)
    gi, _ = run_gpu(q, kc, table, np.array([40 * 64], np.int32), 5, return_physical=True)
    assert np.array_equal(gi[0, 0], [39, 38, 37, 36, 35])


def test_garbage_past_seq_len_is_masked():
    q, kc, table, lens = make_paged_case(303, 1, 32, 8, 4, 128, [300])
    a = run_gpu(q, kc, table, lens, 2)
    kc2 = kc.copy()
    kc2[table[0, 2], 300 - 256:] = q[0, 0]  # perfect matches in the masked tail
    b = run_gpu(q, kc2, table, lens, 2)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_out_of_range_table_entry_scores_minus_one():
    q, kc, table, lens = make_paged_case(304, 1, 32, 8, 4, 128, [512])
    table[0, 1] = kc.shape[0] + 7
    table[0, 3] = -2
    check(q, kc, table, lens, 4)
    gi, gs = run_gpu(q, kc, table, lens, 4)
    assert np.all(gs[0, :, 1] == -1) and np.all(gs[0, :, 3] == -1)


def test_contiguous_cache_without_table():
    rng = rng_for(305)
    kc = random_codes(rng, (2 * 6, 128, 8, 4))
    q = random_codes(rng, (2, 32, 4))
    lens = np.array([700, 768], np.int32)
    table = np.arange(12, dtype=np.int32).reshape(2, 6)
    gi, gs = run_gpu(q, kc, None, lens, 3, max_blocks=6)
    oi, os_ = run_oracle(q, kc, table, lens, 3)
    assert np.array_equal(gi, oi) and np.array_equal(gs, os_)


def test_more_blocks_than_the_lds_row_cap():
    """More than 8192 blocks in one request: selection reads scores from global memory."""
    q, kc, table, lens = make_paged_case(306, 1, 2, 2, 4, 16, [16 * 9000 + 5], extra_blocks=1)
    check(q, kc, table, lens, 33)
    check(q, kc, table, lens, 33, reduce_heads=True)


def test_strided_query_and_table():
    q, kc, table, lens = make_paged_case(307, 2, 32, 8, 4, 128, [900, 300], table_pad=5)
    from ucm_amd.sparse import hamming_topk

    qbig = torch.zeros((2, 40, 6), dtype=torch.int32, device="cuda")
    qbig[:, :32, :4] = dev(as_i32(q))
    tbig = torch.zeros((2, table.shape[1] + 9), dtype=torch.int32, device="cuda")
    tbig[:, : table.shape[1]] = dev(table)
    idx, sc = hamming_topk(qbig[:, :32, :4], dev(as_i32(kc)), tbig[:, : table.shape[1]],
                           dev(lens), 4)
    oi, os_ = run_oracle(q, kc, table, lens, 4)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(sc.cpu().numpy(), os_)


def test_per_token_scores_int32_and_f16():
    from ucm_amd.sparse import hamming_score

    q, kc, table, lens = make_paged_case(308, 2, 32, 8, 4, 128, [700, 1000], table_pad=1)
    msl = table.shape[1] * 128
    for sink, recent, red in ((0, 0, False), (128, 512, True), (3, 5, False)):
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, red)
        g = hamming_score(dev(as_i32(kc)), dev(as_i32(q))[:, None], dev(table), dev(lens), msl,
                          sink, recent, red, out_int32=True).cpu().numpy()
        assert np.array_equal(g, o)
        h = hamming_score(dev(as_i32(kc)), dev(as_i32(q))[:, None], dev(table), dev(lens), msl,
                          sink, recent, red).cpu().numpy()
        expect = np.where(o == c_api.INF, np.inf, o.astype(np.float64)).astype(np.float16)
        assert np.array_equal(h, expect)  # distances <= 512 are exact in half


def test_f16_scores_round_like_sequential_half_adds():
    """128 query heads x 256-bit codes: sums exceed 2048, so half accumulation rounds.  The
    kernel must round like the reference's loop (paged_ham_dist_mla.cu:235-241): one half add
    per 64-bit piece."""
    from ucm_amd.sparse import hamming_score

    q, kc, table, lens = make_paged_case(309, 1, 128, 1, 8, 64, [640])
    msl = table.shape[1] * 64
    h = hamming_score(dev(as_i32(kc)), dev(as_i32(q))[:, None], dev(table), dev(lens), msl,
                      0, 0, False).cpu().numpy()
    # emulate: per 64-bit piece, integer group-summed popcount -> half, accumulate in half
    kpieces = np.ascontiguousarray(kc).view(np.uint64)  # [NB,BS,1,4]
    qpieces = np.ascontiguousarray(q).view(np.uint64)   # [1,128,4]
    expect = np.full((1, 1, msl), np.inf, np.float16)
    for p in range(640):
        pb, t = table[0, p // 64], p % 64
        acc = np.float16(0)
        for c in range(4):
            x = kpieces[pb, t, 0, c] ^ qpieces[0, :, c]
            part = int(sum(bin(int(v)).count("1") for v in x))
            acc = np.float16(acc + np.float16(part))
        expect[0, 0, p] = acc
    assert np.array_equal(h, expect)


@pytest.mark.parametrize("G", [1, 2, 4, 5, 8, 16, 128])
@pytest.mark.parametrize("Wd,BS", [(18, 64), (18, 128), (18, 192), (18, 16), (18, 1), (16, 256), (8, 192),
                                   (6, 32), (2, 64), (34, 8), (64, 4)])
def test_one_kv_head_even_code_widths(G, Wd, BS):
    """One KV head with codes that are not a whole number of 16-byte pieces per token — the
    18-word (512 + 64 bit) codes of the reference's latent-attention path
    (hamming_topk.py: `k_hash.shape[-1] == 18`) and other even widths: block top-k, exact
    per-token distances and the half-precision output against the checker."""
    from ucm_amd.sparse import hamming_score

    lens_list = [BS * 7 + BS // 2 + 1, BS * 21, 1, 0]
    q, kc, table, lens = make_paged_case(400 + G + Wd, 4, G, 1, Wd, BS, lens_list, table_pad=2)
    check(q, kc, table, lens, 5)
    check(q, kc, table, lens, 6, sink=BS, recent=2 * BS, distance=True, score_order=True)
    table[1, 3] = kc.shape[0] + 1  # unusable entry
    check(q, kc, table, lens, 22, return_physical=True)
    msl = table.shape[1] * BS - BS // 2
    args = (dev(as_i32(kc)), dev(as_i32(q))[:, None], dev(table), dev(lens), msl)
    for sink, recent in ((0, 0), (BS + 1, 3)):
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, False)
        g = hamming_score(*args, sink, recent, False, out_int32=True).cpu().numpy()
        assert np.array_equal(g, o)
    h = hamming_score(*args, 0, 0, False).cpu().numpy()
    expect = half_piece_sums(q, kc, table, lens, msl)
    assert np.array_equal(h, expect)


@pytest.mark.parametrize("G,Wd,BS", [(1, 18, 64), (64, 18, 64), (128, 18, 128), (16, 16, 64), (5, 6, 16)])
def test_one_kv_head_contiguous_cache_without_table(G, Wd, BS):
    """The one-KV-head kernels with block j of request b at b * max_blocks + j (no table)."""
    rng = rng_for(450 + G + Wd)
    B, mb = 3, 9
    kc = random_codes(rng, (B * mb, BS, 1, Wd))
    q = random_codes(rng, (B, G, Wd))
    lens = np.array([mb * BS, 4 * BS + 3, 1], np.int32)
    table = np.arange(B * mb, dtype=np.int32).reshape(B, mb)
    for kw in ({}, {"return_physical": True}, {"score_order": True, "distance": True}):
        gi, gs = run_gpu(q, kc, None, lens, 4, max_blocks=mb, **kw)
        oi, os_ = run_oracle(q, kc, table, lens, 4, **kw)
        assert np.array_equal(gi, oi) and np.array_equal(gs, os_)


@pytest.mark.parametrize("S,Hkv,G,Wd", [(1024, 8, 1, 4), (1000, 4, 2, 8), (333, 1, 64, 18), (640, 1, 1, 18)])
def test_per_token_scores_contiguous_form(S, Hkv, G, Wd):
    """block_table=None: key_codes [B, S, Hkv, C], position p of request b at key_codes[b, p]
    (the reference's non-block mode, paged_ham_dist_mla.cu:345,444-)."""
    from ucm_amd.sparse import hamming_score

    rng = rng_for(460 + S)
    B = 3
    kc = random_codes(rng, (B, S, Hkv, Wd))
    q = random_codes(rng, (B, Hkv * G, Wd))
    lens = np.array([S, S // 2 + 1, 0], np.int32)
    # checker: one block of S tokens per request
    table = np.arange(B, dtype=np.int32).reshape(B, 1)
    for red in ((False, True) if Hkv > 1 else (False,)):
        o = c_api.hamming_score(q, kc, table, lens, S, 3, 5, red)
        g = hamming_score(dev(as_i32(kc)), dev(as_i32(q))[:, None], None, dev(lens), S, 3, 5, red,
                          out_int32=True).cpu().numpy()
        assert np.array_equal(g, o)


def test_update_seq_lens():
    from ucm_amd.sparse import update_seq_lens

    lens = np.array([1000, 256, 100, 257, 0, 32768], np.int32)
    out = update_seq_lens(dev(lens), 256, 128).cpu().numpy()
    assert np.array_equal(out, c_api.update_seq_lens(lens, 256, 128))


def test_reference_shaped_wrapper():
    """cuda_hamming_topk (hamming_topk.py:15-54): one physical block list per request."""
    from ucm_amd.sparse import cuda_hamming_topk

    q, kc, table, lens = make_paged_case(310, 2, 8, 8, 4, 128, [5000, 4000], table_pad=2)
    # the plugin hashes the group-mean query: one code per KV head (G = 1)
    out = cuda_hamming_topk(dev(as_i32(q))[:, None], dev(as_i32(kc)), dev(table), dev(lens),
                            topk_token=2048, sink_token=128, recent_token=512, is_mla=False)
    oi, _ = run_oracle(q, kc, table, lens, 16, 128, 512, reduce_heads=True, return_physical=True)
    assert np.array_equal(out.cpu().numpy(), oi[:, 0])


def test_bad_arguments_raise():
    from ucm_amd.sparse import hamming_topk

    q, kc, table, lens = make_paged_case(311, 1, 32, 8, 4, 128, [256])
    with pytest.raises(ValueError):
        hamming_topk(dev(as_i32(q))[:, :30], dev(as_i32(kc)), dev(table), dev(lens), 2)
    with pytest.raises(ValueError):
        hamming_topk(dev(as_i32(q)), dev(as_i32(kc)), dev(table), dev(lens), 0)
    with pytest.raises(ValueError):
        hamming_topk(dev(as_i32(q)), dev(as_i32(kc)), dev(table.astype(np.int64)), dev(lens), 2)

