"""GPU: which kernels a shape takes.  Several kernel families compute the same block scores at
very different speeds, so a dispatch regression to a general kernel would pass every parity test
and only show up as time.  Every family is reached here by a shape of its own, checked
bit-exactly against the CPU checker, and the BASELINE.json shapes are pinned to the kernels
that were tuned for them."""
import numpy as np
import pytest
import torch

from helpers import make_paged_case
from oracle import c_api

pytestmark = pytest.mark.gpu


def _dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.cuda()


# (B, Hq, Hkv, Wd, BS, lens, k, kwargs, kernels launched)
TOPK_SHAPES = {
    "config1": (1, 32, 8, 4, 128, [8192], 16, {}, "block_score_one<1,8,1,4,1>+select_wave_kernel<4>"),
    "config2_two_requests": (2, 32, 8, 4, 128, [32768, 32768], 64, {},
                             "block_score_one<1,8,1,4,1>+select_wave_kernel<4>"),
    "config3_one_long_request": (1, 32, 8, 4, 128, [70001], 128, {},
                                 "block_score_one<1,8,1,4,1>+select_group_kernel<4>"),
    "config5_two_requests": (2, 128, 1, 8, 64, [65536, 700], 128, {},
                             "block_score_strip8+select_group_kernel<4>"),
    "config5_shape_255_query_heads": (2, 255, 1, 8, 64, [4096, 700], 16, {},
                                      "block_score_dot64<2>+select_wave_kernel<4>"),
    "plugin_reduced_physical": (2, 8, 8, 4, 128, [4096, 3000], 8,
                                {"reduce_heads": True, "return_physical": True},
                                "block_score_one<1,8,1,1,1>+select_wave_kernel<4>"),
    "blocks_of_32_KiB": (2, 32, 8, 4, 256, [4096, 3000], 4, {}, "block_score_one<1,8,1,4,0>+select_wave_kernel<4>"),
    "eight_query_heads_per_kv_head": (2, 64, 8, 4, 128, [4096, 3000], 8, {},
                                      "plane_kernel+block_score_one<1,8,0,4,1>+select_wave_kernel<4>"),
    "sixteen_query_heads_per_kv_head": (2, 128, 8, 4, 128, [4096, 3000], 8, {},
                                        "plane_kernel+block_score_one<1,8,0,5,1>+select_wave_kernel<4>"),
    "thirty_one_query_heads_one_kv_head": (2, 31, 1, 4, 1024, [8192, 3000], 4, {},
                                           "plane_kernel+block_score_one<1,1,0,5,1>+select_wave_kernel<4>"),
    "blocks_of_64_tokens": (2, 32, 8, 4, 64, [4096, 3000], 8, {}, "block_score_rows<1,8,4,8>+select_wave_kernel<4>"),
    "blocks_of_16_tokens": (2, 32, 8, 4, 16, [1024, 700], 8, {}, "block_score_rows<1,8,4,2>+select_wave_kernel<4>"),
    "small_blocks_bit_planes": (2, 16, 2, 4, 32, [2048, 700], 8, {},
                                "plane_kernel+block_score_small<1,2,0,4,1>+select_wave_kernel<4>"),
    "odd_block_size_bit_planes": (2, 64, 8, 4, 48, [2048, 700], 8, {},
                                  "plane_kernel+block_score_fast<1,0,4,4>+select_wave_kernel<4>"),
    "blocks_below_1_KiB": (2, 1, 1, 4, 16, [2048, 700], 8, {}, "block_score_tiny<1,1>+select_wave_kernel<4>"),
    "one_head_6_words": (2, 1, 1, 6, 32, [2048, 700], 8, {}, "block_score_pairs<1,1>+select_wave_kernel<4>"),
    "one_head_6_words_16_query_heads": (2, 16, 1, 6, 32, [2048, 700], 8, {},
                                        "plane_kernel+block_score_pairs<0,5>+select_wave_kernel<4>"),
    "latent_18_words": (2, 1, 1, 18, 64, [4096, 700], 8, {}, "block_score_lanes<9,1,1>+select_wave_kernel<4>"),
    "latent_18_words_64_query_heads": (2, 64, 1, 18, 64, [4096, 700], 8, {},
                                       "block_score_strip18+select_wave_kernel<4>"),
    "config5_blocks_of_128": (2, 128, 1, 8, 128, [8192, 700], 8, {},
                              "plane_kernel+block_score_lanes<4,0,8>+select_wave_kernel<4>"),
    "odd_code_width": (2, 6, 2, 3, 16, [1024, 300], 8, {}, "block_score_generic+select_wave_kernel<4>"),
    "more_than_4096_blocks": (1, 4, 1, 4, 16, [70000], 16, {}, "block_score_tiny<1,4>+select_kernel"),
    "score_order": (2, 32, 8, 4, 128, [4096, 3000], 8, {"score_order": True},
                    "block_score_one<1,8,1,4,1>+select_kernel"),
}


@pytest.mark.parametrize("name", list(TOPK_SHAPES))
def test_topk_shape_takes_its_kernels_and_matches_the_checker(name):
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_topk

    B, Hq, Hkv, Wd, BS, lens, k, kw, expect = TOPK_SHAPES[name]
    q, kc, table, lens = make_paged_case(1234, B, Hq, Hkv, Wd, BS, lens)
    idx, sc = hamming_topk(_dev(q), _dev(kc), _dev(table), _dev(lens), k, **kw)
    assert _lib.last_dispatch() == expect
    torch.cuda.synchronize()
    flags = ((c_api.F_REDUCE_HEADS if kw.get("reduce_heads") else 0)
             | (c_api.F_PHYSICAL if kw.get("return_physical") else 0)
             | (c_api.F_SCORE_ORDER if kw.get("score_order") else 0))
    oi, os_ = c_api.hamming_topk(q, kc, table, lens, k, 0, 0, flags)
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.array_equal(sc.cpu().numpy(), os_)


# (B, Hq, Hkv, Wd, BS, lens, kernels launched)
SCORE_SHAPES = {
    "config2_two_requests": (2, 32, 8, 4, 128, [32768, 30000], "token_score_one<4,8>"),
    "config2_codes_in_64_token_blocks": (2, 32, 8, 4, 64, [16384, 9000], "token_score_fast<4>"),
    "config2_codes_two_words_wider": (2, 16, 8, 8, 128, [8192, 3000], "token_score_fast<2>"),
    "one_head_6_words": (2, 2, 1, 6, 32, [2048, 700], "token_score_pairs<1,2>"),
    "one_head_6_words_16_query_heads": (2, 16, 1, 6, 32, [2048, 700], "plane_kernel+token_score_pairs<0,5>"),
    "latent_18_words": (2, 1, 1, 18, 64, [4096, 700], "token_score_lanes<9,1,1>"),
    "latent_18_words_64_query_heads": (2, 64, 1, 18, 64, [4096, 700], "token_score_strip<18,0>"),
    "latent_8_words_128_query_heads": (2, 128, 1, 8, 64, [4096, 700], "token_score_strip<8,0>"),
    "latent_18_words_64_query_heads_128_token_blocks": (2, 64, 1, 18, 128, [4096, 700],
                                                        "plane_kernel+token_score_lanes<9,0,7>"),
    "odd_code_width": (2, 6, 2, 3, 16, [1024, 300], "token_score_kernel"),
}


@pytest.mark.parametrize("name", list(SCORE_SHAPES))
def test_per_token_scorer_takes_its_kernels_and_matches_the_checker(name):
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_score

    B, Hq, Hkv, Wd, BS, lens, expect = SCORE_SHAPES[name]
    q, kc, table, lens = make_paged_case(4321, B, Hq, Hkv, Wd, BS, lens)
    msl = int(max(lens))
    out = hamming_score(_dev(kc), _dev(q), _dev(table), _dev(lens), msl, 0, 0, False, out_int32=True)
    assert _lib.last_dispatch() == expect
    torch.cuda.synchronize()
    ref = c_api.hamming_score(q, kc, table, lens, msl)
    assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("Wd,BS", [(8, 64), (18, 64), (16, 64), (8, 128), (18, 128)])
@pytest.mark.parametrize("G", [3, 5, 8, 15, 16, 31, 33, 48, 49, 64, 100, 127, 128, 200])
def test_planes_built_inside_the_scorer_for_every_group_size(G, Wd, BS):
    """One KV head: the scorer reduces the G query heads to per-bit counts itself (no plane kernel)
    when the blocks hold 64 tokens - for every G with 8-word codes (16 to 128 heads: signed base-4
    digits of G - 2 * count as FP4 operands of the matrix instruction; fewer or more: counts as nibble
    digits for the 4-bit dot product), up to 128 heads with 18-word codes (the matrix instruction
    again) and with 16-word codes (bit planes); larger blocks keep
    the plane kernel.  Ragged lengths (an empty request, a length that ends inside a block, runs
    that end inside a workgroup), table entries out of range, forced blocks."""
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_topk

    lens = [0, 1, 63, 64, 65, 700, 1024 + 17, 5000, 16 * 64 * 3 + 1]
    B = len(lens)
    q, kc, table, lens = make_paged_case(77 + G + Wd, B, G, 1, Wd, BS, lens)
    if G % 2:  # low-entropy queries: many per-bit counts of 0 and of G
        q[:, :, :4] = q[:, :1, :4]
        q[:, :, 4] = 0
        q[:, :, 5] = 0xFFFFFFFF
    table[5, 3] = -1
    table[7, 11] = kc.shape[0] + 5
    k = 9
    planes = max(4, int(G).bit_length())
    for sink, recent in ((0, 0), (64, 256)):
        idx, sc = hamming_topk(_dev(q), _dev(kc), _dev(table), _dev(lens), k, sink, recent)
        got = _lib.last_dispatch()
        if (Wd, BS) == (8, 64):
            if 16 <= G <= 128:
                assert got.startswith("block_score_strip8+")
            else:
                assert got.startswith("block_score_dot64<%d>+" % (1 if G <= 15 else 2))
        elif (Wd, BS) == (18, 64) and G <= 128:
            assert got.startswith("block_score_strip18+")
        elif BS == 64 and G <= 128:
            assert got.startswith("block_score_lanes_run<%d,%d>+" % (Wd // 2, planes))
        else:
            assert got.startswith("plane_kernel+block_score_lanes<%d,0,%d>+" % (Wd // 2, min(planes, 8)))
        torch.cuda.synchronize()
        oi, os_ = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, 0)
        assert np.array_equal(sc.cpu().numpy(), os_)
        assert np.array_equal(idx.cpu().numpy(), oi)


@pytest.mark.parametrize("Wd,G", [(18, 3), (18, 63), (18, 64), (18, 112), (18, 127), (18, 128),
                                  (8, 16), (8, 63), (8, 64), (8, 127), (8, 128)])
def test_latent_18_word_scorer_extreme_weights(Wd, G):
    """The latent scorers (18-word and 8-word codes) multiply code bits with signed weights G - 2 * count
    on the matrix unit (FP4 operands, float accumulation) and must stay exact at the ends of their range:
    every query head equal (all counts 0 or G, weights of magnitude G, up to 128), all-ones and all-zero
    cached codes (the largest sums), one bit set per word, and a run of blocks that ends inside a
    workgroup's run with a last block of a single token - block scores, and the per-token mode's int32
    distances and half-precision sums (paged_ham_dist_mla.cu:235-241)."""
    from helpers import half_piece_sums
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_score, hamming_topk

    lens = [64 * 9 + 1, 64 * 40, 17]
    q, kc, table, lens = make_paged_case(900 + G + Wd, len(lens), G, 1, Wd, 64, lens)
    half = Wd // 2
    q[0, :, :] = q[0, :1, :]              # request 0: all heads equal
    q[1, : G // 2, :] = 0xFFFFFFFF        # request 1: counts of G // 2 or G everywhere
    q[1, G // 2:, :half] = 0
    q[1, G // 2:, half:] = 0xFFFFFFFF
    nb = kc.shape[0]
    kc[0::5] = 0xFFFFFFFF                 # whole blocks of all-ones / all-zero codes
    kc[1::5] = 0
    kc[2::5, ::2] = 0x80000001            # bits 0 and 31 of every word
    kc[2::5, 1::2] = 0x00011000
    assert nb >= 5
    for sink, recent in ((0, 0), (64, 64)):
        idx, sc = hamming_topk(_dev(q), _dev(kc), _dev(table), _dev(lens), 12, sink, recent)
        assert _lib.last_dispatch().startswith("block_score_strip%d+" % Wd)
        torch.cuda.synchronize()
        oi, os_ = c_api.hamming_topk(q, kc, table, lens, 12, sink, recent, 0)
        assert np.array_equal(sc.cpu().numpy(), os_)
        assert np.array_equal(idx.cpu().numpy(), oi)
        msl = 64 * 40
        tok = hamming_score(_dev(kc), _dev(q), _dev(table), _dev(lens), msl, sink, recent, False, out_int32=True)
        assert _lib.last_dispatch() == "token_score_strip<%d,0>" % Wd
        assert np.array_equal(tok.cpu().numpy(), c_api.hamming_score(q, kc, table, lens, msl, sink, recent, False))
    h = hamming_score(_dev(kc), _dev(q), _dev(table), _dev(lens), 64 * 40, 0, 0, False).cpu().numpy()
    assert np.array_equal(h, half_piece_sums(q, kc, table, lens, 64 * 40))


@pytest.mark.parametrize("Wd,G", [(18, 64), (8, 128)])
def test_latent_scorer_clock_probe(Wd, G):
    """The measurement aid of the latent scorers: with a probe address set, the last wave of the first
    workgroup reports the shader cycles and the 100 MHz ticks of its life (a plausible clock), in the block
    scorer and in its per-token mode; results are the same with and without it; a misaligned address is
    refused."""
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_score, hamming_topk

    L = _lib.lib()
    q, kc, table, lens = make_paged_case(99 + Wd, 2, G, 1, Wd, 64, [8192, 700])
    args = (_dev(q), _dev(kc), _dev(table), _dev(lens), 16)
    ref_idx, ref_sc = hamming_topk(*args)
    ref_tok = hamming_score(_dev(kc), _dev(q), _dev(table), _dev(lens), 8192, 0, 0, False)
    probe = torch.zeros(2, dtype=torch.int64, device="cuda")
    _lib.check(L.ucm_hamming_topk_set_clock_probe(probe.data_ptr()))
    try:
        for mode in ("blocks", "tokens"):
            probe.zero_()
            if mode == "blocks":
                idx, sc = hamming_topk(*args)
                assert _lib.last_dispatch().startswith("block_score_strip%d+" % Wd)
                assert torch.equal(idx, ref_idx) and torch.equal(sc, ref_sc)
            else:
                tok = hamming_score(_dev(kc), _dev(q), _dev(table), _dev(lens), 8192, 0, 0, False)
                assert _lib.last_dispatch() == "token_score_strip<%d,1>" % Wd
                assert torch.equal(tok, ref_tok)
            torch.cuda.synchronize()
            cycles, ticks = (int(v) for v in probe.cpu().tolist())
            assert cycles > 1000 and ticks > 10, (mode, cycles, ticks)
            assert 0.3 < cycles / (ticks * 10.0) < 3.5, (mode, cycles, ticks)
        assert L.ucm_hamming_topk_set_clock_probe(probe.data_ptr() + 4) == _lib.UCM_EPARAM
    finally:
        _lib.check(L.ucm_hamming_topk_set_clock_probe(None))
