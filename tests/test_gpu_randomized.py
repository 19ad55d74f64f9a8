"""Randomised differential tests (fixed seeds): many small random configurations of the scorer /
top-k and of the encoder's three paths against the CPU checker.  The hand-picked cases elsewhere
aim at known corners; these sweep combinations nobody thought of.  Bit-exact for the top-k, the
margin rule (|projection| < 1e-2 * ||x||) for hash bits."""
import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import brute, c_api

pytestmark = pytest.mark.gpu

MARGIN_TOL = 1e-2


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_topk_random_configurations(seed):
    from ucm_amd.sparse import hamming_topk

    rng = rng_for(seed)
    for _ in range(250):
        B = int(rng.integers(1, 7))
        Hkv = int(rng.choice([1, 2, 3, 4, 8]))
        G = int(rng.choice([1, 2, 3, 4, 8, 16]))
        Wd = int(rng.choice([1, 2, 4, 6, 8]))
        BS = int(rng.choice([4, 8, 16, 32, 64, 128]))
        mb = int(rng.integers(1, 200))
        NB = B * mb + int(rng.integers(0, 5))
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, Wd), dtype=np.uint32)
        if rng.integers(0, 4) == 0:
            kc &= np.uint32(0x01010101)  # low-entropy codes: many equal scores
        q = rng.integers(0, 2**32, size=(B, Hkv * G, Wd), dtype=np.uint32)
        use_table = bool(rng.integers(0, 4))
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32) if use_table else None
        if not use_table:
            kc = kc[:B * mb]
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        if rng.integers(0, 3) == 0:
            lens[rng.integers(0, B)] = mb * BS
        k = int(rng.integers(1, min(mb, 128) + 3))
        sink = int(rng.integers(0, 3)) * BS if rng.integers(0, 3) == 0 else 0
        recent = int(rng.integers(0, 3)) * BS if rng.integers(0, 3) == 0 else 0
        reduce_heads, physical = bool(rng.integers(0, 4) == 0), bool(rng.integers(0, 3) == 0)
        score_order, distance = bool(rng.integers(0, 3) == 0), bool(rng.integers(0, 3) == 0)
        flags = (c_api.F_REDUCE_HEADS if reduce_heads else 0) | (c_api.F_PHYSICAL if physical else 0) | \
                (c_api.F_SCORE_ORDER if score_order else 0) | (c_api.F_DISTANCE if distance else 0)
        what = dict(B=B, Hkv=Hkv, G=G, Wd=Wd, BS=BS, mb=mb, k=k, table=use_table, sink=sink, recent=recent,
                    flags=flags)
        oi, osc = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=mb)
        gi, gs = hamming_topk(torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda(),
                              torch.from_numpy(table).cuda() if use_table else None, torch.from_numpy(lens).cuda(),
                              k, sink, recent, reduce_heads=reduce_heads, return_physical=physical,
                              score_order=score_order, distance=distance, max_blocks=mb)
        assert np.array_equal(gi.cpu().numpy(), oi), what
        assert np.array_equal(gs.cpu().numpy(), osc), what


def _codes_ok(codes_u8, x32, W32):
    ref = brute.hash_encode(x32, W32).view(np.uint8)
    got = np.ascontiguousarray(codes_u8)
    if np.array_equal(got, ref):
        return True
    diff = np.unpackbits(got ^ ref, axis=-1, bitorder="little").astype(bool)
    return not np.any(diff & (brute.margins(x32, W32) >= MARGIN_TOL))


@pytest.mark.parametrize("seed", [21, 22])
def test_encoder_random_configurations(seed):
    from ucm_amd.sparse import HashEncoder

    rng = rng_for(seed)
    for _ in range(30):
        dt = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        K = int(rng.choice([40, 64, 96, 128, 256, 512]))
        N = int(rng.choice([32, 64, 96, 128, 256, 512]))
        H = int(rng.choice([1, 2, 4, 8]))
        T = int(rng.choice([1, 3, 31, 32, 33, 100, 257, 511, 1024, 1500, 4096]))
        n_w = int(rng.choice([1, H]))
        BS = int(rng.choice([8, 16, 32, 64, 128]))
        what = dict(dt=str(dt), K=K, N=N, H=H, T=T, n_w=n_w, BS=BS)
        W = torch.from_numpy(rng.standard_normal((n_w, K, N)).astype(np.float32)).to(dt)
        enc = HashEncoder(K, N, dt, torch.device("cuda:0"), num_weights=n_w, heads_per_weight=1)
        enc.set_hash_weight(W.cuda() if n_w > 1 else W[0].cuda())
        x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(dt)
        if rng.integers(0, 5) == 0:
            x[rng.integers(0, T)] = 0
        W32, x32 = W.float().numpy(), x.float().numpy()
        # dense, one matrix per head
        codes = enc.compute_hash(x.cuda(), per_head=True).cpu().numpy()
        for h in range(H):
            assert _codes_ok(codes[:, h], x32[:, h], W32[min(h, n_w - 1)]), ("dense", what, h)
        # paged store through a random slot mapping, a tenth of the rows dropped
        NBc = (T + BS - 1) // BS + 2
        slots = rng.permutation(NBc * BS)[:T].astype(np.int64)
        drop = rng.random(T) < 0.1
        slots_d = np.where(drop, -1, slots)
        cache = torch.full((NBc, BS, H, N // 32), -1, dtype=torch.int32, device="cuda")
        enc.compute_hash_and_cache(x.cuda(), torch.from_numpy(slots_d).cuda(), cache, BS)
        c = cache.cpu().numpy().view(np.uint8).reshape(NBc * BS, H, N // 8)
        for h in range(H):
            assert _codes_ok(c[slots[~drop], h], x32[~drop, h], W32[min(h, n_w - 1)]), ("paged", what, h)
            assert np.all(c[slots[drop], h] == 0xff), ("dropped slot written", what, h)
        # paged input (prefix-cache rehash)
        nblk = (T + BS - 1) // BS
        kcache = torch.zeros((nblk + 3, BS, H, K), dtype=dt)
        ids = rng.permutation(nblk + 3)[:nblk].astype(np.int32)
        pos = (torch.from_numpy(ids).long().repeat_interleave(BS) * BS + torch.arange(BS).repeat(nblk))[:T]
        kcache.view(-1, H, K)[pos] = x
        codes2 = torch.full((nblk + 3, BS, H, N // 32), -1, dtype=torch.int32, device="cuda")
        enc.compute_hash_from_paged_cache(kcache.cuda(), torch.from_numpy(ids).cuda(), T, codes2, BS)
        c2 = codes2.cpu().numpy().view(np.uint8).reshape(-1, H, N // 8)
        for h in range(H):
            assert _codes_ok(c2[pos.numpy(), h], x32[:, h], W32[min(h, n_w - 1)]), ("rehash", what, h)


@pytest.mark.parametrize("seed", [31, 32])
def test_float_retrieval_random_configurations(seed):
    """KVStar and ESA top-k on random shapes (matrix-core and scalar q.k paths, pruning, the
    counting / bucket / merge selection paths, holes in the candidate lists, rounded data for
    ties) against the checker, with the tolerances of test_gpu_kvstar.py and
    test_gpu_esa_retrieval.py."""
    from ucm_amd.sparse import kvstar_retrieve
    from ucm_amd.sparse.esa_retrieval_worker import dot_topk

    rng = rng_for(seed)
    for _ in range(40):
        Hkv, g = int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 4, 7]))
        Hq, X = Hkv * g, int(rng.integers(1, 12))
        d, M = int(rng.choice([8, 16, 20, 32, 48, 64, 128])), int(rng.choice([1, 2, 3, 4]))
        n = int(rng.integers(1, 1200))
        n = min(n, max(1, 1_500_000 // (M * X * Hq)))
        topk = int(rng.integers(1, min(n, 200) + 2))
        pr, d_orig = None, d
        if rng.integers(0, 3) == 0:
            d_orig = d + int(rng.integers(1, 40))
            pr = np.stack([np.sort(rng.permutation(d_orig)[:d]) for _ in range(Hkv)]).astype(np.int64)
        q = (rng.standard_normal((X, Hq, d_orig)) * 0.5).astype(np.float16)
        k = (rng.standard_normal((n, M, Hkv, d)) * 0.5).astype(np.float16)
        what = dict(X=X, Hq=Hq, Hkv=Hkv, d=d, d_orig=d_orig, n=n, M=M, topk=topk)
        gi, gs = kvstar_retrieve.kvstar_topk(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(),
                                              torch.from_numpy(pr).cuda() if pr is not None else None, topk)
        gi, gs = gi.cpu().numpy().astype(np.int64), gs.cpu().numpy()
        oi, osc, allsc = c_api.kvstar_topk(q, k, topk, pr)
        tol = 1e-7 + 2e-5 * np.abs(osc)
        assert gi.shape == oi.shape and len(set(gi.tolist())) == gi.size, what
        assert np.all(np.abs(gs - osc) <= tol), what
        for t in np.nonzero(gi != oi)[0]:
            assert abs(allsc[gi[t]] - allsc[oi[t]]) <= 2 * tol[t], what

        n_items, dim = int(rng.integers(10, 12000)), int(rng.choice([16, 30, 64, 100, 256, 1024]))
        B = int(rng.integers(1, 4))
        max_n = int(rng.integers(1, min(n_items, 10000) + 1))
        kk = int(rng.integers(1, min(max_n, 4096) + 1))
        data = rng.standard_normal((n_items, dim)).astype(np.float32)
        query = rng.standard_normal((B, dim)).astype(np.float32)
        if rng.integers(0, 4) == 0:
            data, query = np.round(data), np.round(query)  # exact scores, many ties
        idx = np.stack([rng.permutation(n_items)[:max_n] for _ in range(B)]).astype(np.int32)
        idx[rng.random(idx.shape) < 0.05] = -1
        what = dict(n_items=n_items, dim=dim, B=B, max_n=max_n, k=kk)
        gi, gs = dot_topk(torch.from_numpy(data).cuda(), torch.from_numpy(query).cuda(),
                          torch.from_numpy(idx).cuda(), kk)
        gi, gs = gi.cpu().numpy(), gs.cpu().numpy()
        oi, osc = c_api.dot_topk(data, query, idx, kk)
        exact = query.astype(np.float64) @ data.astype(np.float64).T
        for b in range(B):
            tolb = 1e-5 * (np.abs(query[b].astype(np.float64))[None, :] * np.abs(data.astype(np.float64))).sum(-1)
            valid = oi[b] >= 0
            assert np.array_equal(valid, gi[b] >= 0), what
            assert len(set(gi[b][valid].tolist())) == valid.sum(), what
            assert np.all(np.abs(gs[b][valid] - osc[b][valid]) <= 2 * tolb[oi[b][valid]].max() + 1e-30), what
            for t in np.nonzero(valid & (gi[b] != oi[b]))[0]:
                assert abs(exact[b, gi[b, t]] - exact[b, oi[b, t]]) <= 2 * max(tolb[gi[b, t]], tolb[oi[b, t]]) + 1e-30, what


@pytest.mark.parametrize("seed", [41, 42])
def test_block_transfer_random_configurations(seed):
    """Scatter / gather / batch copies with random chunk sizes (odd ones included), counts,
    permutations, both stream kinds and both directions; every byte compared, and the bytes a
    transfer must not touch checked for their fill value."""
    from ucm_amd.trans import Device

    dev = Device()
    dev.Setup(0)
    rng = rng_for(seed)
    for _ in range(40):
        size = int(rng.choice([1, 3, 16, 100, 4096, 4097, 36 * 1024, 65536 + 8, 262144]))
        number = int(rng.integers(1, 400))
        number = min(number, max(1, (32 << 20) // size))
        stream = dev.MakeSMStream() if rng.integers(0, 2) else dev.MakeStream()
        what = dict(size=size, number=number)
        spare = int(rng.integers(0, 4))
        pool = torch.full((size * (number + spare),), 0xA5, dtype=torch.uint8, device="cuda")
        perm = rng.permutation(number + spare)[:number]
        table = np.array([pool.data_ptr() + int(i) * size for i in perm], dtype=np.uint64)
        h1 = torch.empty(size * number, dtype=torch.uint8).pin_memory()
        h1.numpy()[:] = rng.integers(0, 256, size=size * number, dtype=np.uint8)
        h2 = torch.zeros(size * number, dtype=torch.uint8).pin_memory()
        torch.cuda.synchronize()
        stream.HostToDeviceScatterAsync(h1.data_ptr(), table, size, number)
        stream.DeviceToHostGatherAsync(table, h2.data_ptr(), size, number)
        stream.Synchronized()
        assert np.array_equal(h2.numpy(), h1.numpy()), what
        got = pool.cpu().numpy().reshape(number + spare, size)
        assert np.array_equal(got[perm], h1.numpy().reshape(number, size)), what
        untouched = np.setdiff1d(np.arange(number + spare), perm)
        assert np.all(got[untouched] == 0xA5), what
        # chunk-to-chunk batch: device chunks to separately placed host chunks and back
        h3 = torch.zeros(size * number, dtype=torch.uint8).pin_memory()
        hperm = rng.permutation(number)
        htable = np.array([h3.data_ptr() + int(i) * size for i in hperm], dtype=np.uint64)
        stream.DeviceToHostBatchAsync(table, htable, size, number)
        stream.Synchronized()
        assert np.array_equal(h3.numpy().reshape(number, size)[hperm], h1.numpy().reshape(number, size)), what
        pool2 = torch.zeros(size * number, dtype=torch.uint8, device="cuda")
        table2 = np.array([pool2.data_ptr() + int(i) * size for i in range(number)], dtype=np.uint64)
        stream.HostToDeviceBatchAsync(htable, table2, size, number)
        stream.Synchronized()
        assert np.array_equal(pool2.cpu().numpy(), h1.numpy()), what
        stream.close()


@pytest.mark.parametrize("seed", [51, 52])
def test_per_token_scores_random_configurations(seed):
    """The per-token scorer (coalesced kernel and general kernel) against the checker: exact
    int32 distances, and fp16 output wherever the distances stay exactly representable."""
    from ucm_amd.sparse import hamming_score

    rng = rng_for(seed)
    for _ in range(120):
        B = int(rng.integers(1, 5))
        Hkv = int(rng.choice([1, 2, 3, 4, 8]))
        G = int(rng.choice([1, 2, 3, 4, 8]))
        Wd = int(rng.choice([2, 4, 6, 8, 16]))
        BS = int(rng.choice([4, 16, 32, 64, 128]))
        mb = int(rng.integers(1, 40))
        NB = B * mb + 3
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, Wd), dtype=np.uint32)
        q = rng.integers(0, 2**32, size=(B, Hkv * G, Wd), dtype=np.uint32)
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 4) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = NB + 7  # unusable entry
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        msl = mb * BS - int(rng.integers(0, BS))
        msl = max(msl, 1)
        sink, recent = int(rng.integers(0, 2 * BS)), int(rng.integers(0, 2 * BS))
        red = bool(rng.integers(0, 4) == 0)
        what = dict(B=B, Hkv=Hkv, G=G, Wd=Wd, BS=BS, mb=mb, msl=msl, sink=sink, recent=recent, red=red)
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, red)
        args = (torch.from_numpy(kc.view(np.int32)).cuda(), torch.from_numpy(q.view(np.int32)).cuda()[:, None],
                torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda(), msl, sink, recent, red)
        g = hamming_score(*args, out_int32=True).cpu().numpy()
        assert np.array_equal(g, o), what
        if G * Wd * 32 <= 2048:
            h = hamming_score(*args).cpu().numpy()
            expect = np.where(o == c_api.INF, np.inf, o.astype(np.float64)).astype(np.float16)
            assert np.array_equal(h, expect), what


@pytest.mark.parametrize("seed", [55, 56])
def test_per_token_scores_16_kib_blocks_random_configurations(seed):
    """The per-token kernel of the hot shape (128-bit codes, blocks of exactly 16 KiB, row length a multiple
    of four) against the checker: lengths that end inside a block, unusable table entries, sink and recent
    windows that cut blocks, rows that end before or reach past the last table entry, both output types,
    with and without the KV-head reduction."""
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_score

    rng = rng_for(seed)
    for it in range(60):
        B = int(rng.integers(1, 5))
        Hkv, BS = (8, 128) if rng.integers(0, 2) else (4, 256)
        G = int(rng.choice([1, 2, 4, 8]))
        mb = int(rng.integers(1, 24))
        NB = B * mb + 3
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, 4), dtype=np.uint32)
        q = rng.integers(0, 2**32, size=(B, Hkv * G, 4), dtype=np.uint32)
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 3) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = NB + 7 if rng.integers(0, 2) else -1
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        if it % 7 == 0:
            lens[0] = mb * BS
        msl = max(4, mb * BS - 4 * int(rng.integers(0, BS // 4)))
        if it % 5 == 0:
            msl = mb * BS + 4 * int(rng.integers(1, BS))  # the row reaches past the last table entry
        sink, recent = int(rng.integers(0, 3 * BS)), int(rng.integers(0, 3 * BS))
        red = bool(rng.integers(0, 3) == 0)
        what = dict(B=B, Hkv=Hkv, G=G, BS=BS, mb=mb, msl=msl, sink=sink, recent=recent, red=red, lens=lens.tolist())
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, red)
        args = (torch.from_numpy(kc.view(np.int32)).cuda(), torch.from_numpy(q.view(np.int32)).cuda()[:, None],
                torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda(), msl, sink, recent, red)
        g = hamming_score(*args, out_int32=True).cpu().numpy()
        assert _lib.last_dispatch() == "token_score_one<%d,%d>" % (G, Hkv), what
        assert np.array_equal(g, o), what
        h = hamming_score(*args).cpu().numpy()
        expect = np.where(o == c_api.INF, np.inf, o.astype(np.float64)).astype(np.float16)
        assert np.array_equal(h, expect), what


@pytest.mark.parametrize("seed", [61, 62])
def test_one_kv_head_random_configurations(seed):
    """One KV head (the latent-attention layout) with even and odd code widths and up to 255 query
    heads: block top-k, exact per-token distances, and the half-precision output against the
    reference's piecewise accumulation (paged_ham_dist_mla.cu:235-241)."""
    from helpers import half_piece_sums
    from ucm_amd.sparse import hamming_score, hamming_topk

    rng = rng_for(seed)
    for _ in range(60):
        B = int(rng.integers(1, 5))
        G = int(rng.choice([1, 2, 3, 4, 8, 16, 64, 128, 255]))
        Wd = int(rng.choice([2, 3, 6, 8, 10, 16, 18, 34]))
        BS = int(rng.choice([1, 4, 16, 64, 128]))
        mb = int(rng.integers(1, 30))
        NB = B * mb + 3
        kc = rng.integers(0, 2**32, size=(NB, BS, 1, Wd), dtype=np.uint32)
        if rng.integers(0, 4) == 0:
            kc &= np.uint32(0x00010001)  # low-entropy codes: many equal scores
        q = rng.integers(0, 2**32, size=(B, G, Wd), dtype=np.uint32)
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 4) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = NB + 7  # unusable entry
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        if rng.integers(0, 3) == 0:
            lens[rng.integers(0, B)] = mb * BS
        k = int(rng.integers(1, mb + 3))
        sink, recent = int(rng.integers(0, 2 * BS)), int(rng.integers(0, 2 * BS))
        score_order, distance = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        flags = (c_api.F_SCORE_ORDER if score_order else 0) | (c_api.F_DISTANCE if distance else 0)
        what = dict(B=B, G=G, Wd=Wd, BS=BS, mb=mb, k=k, sink=sink, recent=recent, flags=flags)
        dq, dk = torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda()
        dt, dl = torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda()
        oi, osc = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=mb)
        gi, gs = hamming_topk(dq, dk, dt, dl, k, sink, recent, score_order=score_order, distance=distance,
                              max_blocks=mb)
        assert np.array_equal(gi.cpu().numpy(), oi), what
        assert np.array_equal(gs.cpu().numpy(), osc), what
        msl = max(mb * BS - int(rng.integers(0, BS)), 1)
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, False)
        g = hamming_score(dk, dq[:, None], dt, dl, msl, sink, recent, False, out_int32=True).cpu().numpy()
        assert np.array_equal(g, o), what
        if Wd % 2 == 0:
            h = hamming_score(dk, dq[:, None], dt, dl, msl, 0, 0, False).cpu().numpy()
            assert np.array_equal(h, half_piece_sums(q, kc, table, lens, msl)), what


@pytest.mark.parametrize("seed", [65, 66])
def test_latent_per_token_scores_weights_built_in_the_scorer(seed):
    """18-word codes in 64-token blocks with 3 to 128 query heads and 8-word codes with 16 to 128: the per-token
    kernel that builds its weights itself and sums every 8-byte piece on the matrix unit (no plane kernel, no
    workspace), exact int32 distances against the checker and the half-precision output against the
    reference's piecewise accumulation (paged_ham_dist_mla.cu:235-241); lengths that end inside a block,
    unusable table entries, sink and recent windows, rows that end inside a block or reach past the table,
    row lengths that are and are not multiples of four."""
    from helpers import half_piece_sums
    from ucm_amd import _lib
    from ucm_amd.sparse import hamming_score

    rng = rng_for(seed)
    for it in range(40):
        B = int(rng.integers(1, 5))
        Wd = 18 if it % 3 else 8
        G = int(rng.choice([3, 5, 7, 8, 15, 16, 31, 33, 64, 100, 127, 128] if Wd == 18 else [16, 31, 33, 64, 100, 127, 128]))
        mb = int(rng.integers(1, 40))
        NB = B * mb + 3
        kc = rng.integers(0, 2**32, size=(NB, 64, 1, Wd), dtype=np.uint32)
        q = rng.integers(0, 2**32, size=(B, G, Wd), dtype=np.uint32)
        if it % 6 == 0:
            q[:] = q[:, :1]                      # all heads equal: the counts reach G
        if it % 9 == 0:
            kc[:] = 0xFFFFFFFF
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 3) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = NB + 7 if rng.integers(0, 2) else -1
        lens = rng.integers(0, mb * 64 + 1, size=B).astype(np.int32)
        if it % 4 == 0:
            lens[0] = mb * 64
        msl = max(mb * 64 - int(rng.integers(0, 64)), 1)
        if it % 5 == 0:
            msl = mb * 64 + int(rng.integers(1, 200))  # the row reaches past the last table entry
        if it % 2 == 0:
            msl = max(4, msl & ~3)                      # whole groups of four positions: the 8- and 16-byte stores
        sink, recent = int(rng.integers(0, 130)), int(rng.integers(0, 130))
        what = dict(B=B, G=G, Wd=Wd, mb=mb, msl=msl, sink=sink, recent=recent, lens=lens.tolist())
        dq, dk = torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda()
        dt, dl = torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda()
        o = c_api.hamming_score(q, kc, table, lens, msl, sink, recent, False)
        g = hamming_score(dk, dq[:, None], dt, dl, msl, sink, recent, False, out_int32=True).cpu().numpy()
        assert _lib.last_dispatch() == "token_score_strip<%d,0>" % Wd, (_lib.last_dispatch(), what)
        assert np.array_equal(g, o), what
        h = hamming_score(dk, dq[:, None], dt, dl, msl, 0, 0, False).cpu().numpy()
        assert np.array_equal(h, half_piece_sums(q, kc, table, lens, msl)), what


@pytest.mark.parametrize("seed", [71, 72])
def test_topk_rows_of_257_to_4096_blocks(seed):
    """Rows of 257 to 4096 blocks take the workgroup-per-row selection: ragged lengths, ties
    (low-entropy codes), every output flag, head reduction, k up to the row length."""
    from ucm_amd.sparse import hamming_topk

    rng = rng_for(seed)
    for _ in range(40):
        B = int(rng.integers(1, 4))
        Hkv = int(rng.choice([1, 2, 8]))
        G = int(rng.choice([1, 4, 16]))
        Wd = int(rng.choice([2, 4, 18])) if Hkv == 1 else 4
        BS = int(rng.choice([4, 8, 16]))
        mb = int(rng.choice([257, 300, 511, 512, 513, 777, 1000, 1023, 1024, 1025, 2048, 2500, 4096]))
        NB = B * mb + 2
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, Wd), dtype=np.uint32)
        if rng.integers(0, 2) == 0:
            kc &= np.uint32(0x00000101)  # many equal scores
        q = rng.integers(0, 2**32, size=(B, Hkv * G, Wd), dtype=np.uint32)
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 3) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = -5  # unusable entry
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        lens[rng.integers(0, B)] = mb * BS - int(rng.integers(0, BS))
        k = int(rng.choice([1, 7, 64, 128, 300, mb, mb + 5]))
        sink, recent = int(rng.integers(0, 3)) * BS, int(rng.integers(0, 5)) * BS
        reduce_heads, physical = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        distance = bool(rng.integers(0, 2))
        flags = (c_api.F_REDUCE_HEADS if reduce_heads else 0) | (c_api.F_PHYSICAL if physical else 0) | \
                (c_api.F_DISTANCE if distance else 0)
        what = dict(B=B, Hkv=Hkv, G=G, Wd=Wd, BS=BS, mb=mb, k=k, sink=sink, recent=recent, flags=flags)
        oi, osc = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=mb)
        gi, gs = hamming_topk(torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda(),
                              torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda(), k, sink, recent,
                              reduce_heads=reduce_heads, return_physical=physical, distance=distance,
                              max_blocks=mb)
        assert np.array_equal(gi.cpu().numpy(), oi), what
        assert np.array_equal(gs.cpu().numpy(), osc), what


@pytest.mark.parametrize("seed", [81, 82])
def test_topk_blocks_below_one_kib(seed):
    """Blocks of 128 to 512 bytes of codes (e.g. 16-token blocks of one or two KV heads, what a
    tensor-parallel rank sees with small serving blocks): several blocks share a wave's run of 64
    pieces, each read through its own table entry.  Rows long enough for several workgroups,
    ragged ends inside a run, unusable table entries, every output flag."""
    from ucm_amd.sparse import hamming_topk

    rng = rng_for(seed)
    for _ in range(60):
        Wd = int(rng.choice([4, 8, 16]))
        cpu = Wd // 4
        Hkv = int(rng.choice([h for h in (1, 2, 4, 8) if h * cpu <= 32]))
        # 8 <= BS * Hkv * cpu < 64 sixteen-byte pieces per block
        BS = int(rng.choice([bs for bs in (1, 2, 4, 8, 16, 32) if 8 <= bs * Hkv * cpu < 64]))
        G = int(rng.choice([1, 2, 4]))
        B = int(rng.integers(1, 5))
        mb = int(rng.choice([1, 3, 15, 16, 17, 63, 64, 65, 127, 129, 255, 300, 700, 1500]))
        NB = B * mb + 3
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, Wd), dtype=np.uint32)
        if rng.integers(0, 3) == 0:
            kc &= np.uint32(0x00010001)  # many equal scores
        q = rng.integers(0, 2**32, size=(B, Hkv * G, Wd), dtype=np.uint32)
        use_table = bool(rng.integers(0, 4))
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32) if use_table else None
        if use_table and rng.integers(0, 3) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = int(rng.choice([-3, NB, NB + 9]))  # unusable entry
        if not use_table:
            kc = kc[:B * mb]
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        lens[rng.integers(0, B)] = mb * BS - int(rng.integers(0, BS))
        k = int(rng.choice([1, 5, 64, mb, mb + 2]))
        sink, recent = int(rng.integers(0, 3)) * BS, int(rng.integers(0, 5)) * BS
        reduce_heads, physical = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        distance = bool(rng.integers(0, 2))
        flags = (c_api.F_REDUCE_HEADS if reduce_heads else 0) | (c_api.F_PHYSICAL if physical else 0) | \
                (c_api.F_DISTANCE if distance else 0)
        what = dict(B=B, Hkv=Hkv, G=G, Wd=Wd, BS=BS, mb=mb, k=k, table=use_table, sink=sink, recent=recent,
                    flags=flags)
        oi, osc = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=mb)
        gi, gs = hamming_topk(torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda(),
                              torch.from_numpy(table).cuda() if use_table else None, torch.from_numpy(lens).cuda(),
                              k, sink, recent, reduce_heads=reduce_heads, return_physical=physical,
                              distance=distance, max_blocks=mb)
        assert np.array_equal(gi.cpu().numpy(), oi), what
        assert np.array_equal(gs.cpu().numpy(), osc), what


@pytest.mark.parametrize("seed", [91])
def test_blocks_of_4_kib_and_more_in_rows_of_over_256_blocks(seed):
    """Blocks of at least 4 KiB (one workgroup per block) in rows of 257 to 1100 blocks (one
    workgroup per row in the selection).  Ragged lengths, ties, unusable entries, every index-ordered flag combination."""
    from ucm_amd.sparse import hamming_topk

    rng = rng_for(seed)
    for _ in range(16):
        Hkv = int(rng.choice([2, 4, 8]))
        Wd, G = 4, int(rng.choice([1, 4, 8]))
        BS = int(rng.choice([bs for bs in (32, 64, 128, 256) if bs * Hkv * 16 >= 4096]))
        B = int(rng.integers(1, 3))
        mb = int(rng.choice([257, 300, 512, 600, 1025, 1100]))
        while B * mb * BS * Hkv * 16 > (48 << 20):
            mb = 257 if mb > 300 else mb
            BS //= 2
        if BS * Hkv * 16 < 4096:
            continue
        NB = B * mb + 2
        kc = rng.integers(0, 2**32, size=(NB, BS, Hkv, Wd), dtype=np.uint32)
        if rng.integers(0, 2) == 0:
            kc &= np.uint32(0x00000101)  # many equal scores
        q = rng.integers(0, 2**32, size=(B, Hkv * G, Wd), dtype=np.uint32)
        table = np.stack([rng.permutation(NB)[:mb] for _ in range(B)]).astype(np.int32)
        if rng.integers(0, 2) == 0:
            table[rng.integers(0, B), rng.integers(0, mb)] = NB + 3  # unusable entry
        lens = rng.integers(0, mb * BS + 1, size=B).astype(np.int32)
        lens[rng.integers(0, B)] = mb * BS - int(rng.integers(0, BS))
        k = int(rng.choice([1, 64, 128, 300, mb]))
        sink, recent = int(rng.integers(0, 3)) * BS, int(rng.integers(0, 5)) * BS
        reduce_heads, physical = bool(rng.integers(0, 3) == 0), bool(rng.integers(0, 2))
        distance = bool(rng.integers(0, 2))
        flags = (c_api.F_REDUCE_HEADS if reduce_heads else 0) | (c_api.F_PHYSICAL if physical else 0) | \
                (c_api.F_DISTANCE if distance else 0)
        what = dict(B=B, Hkv=Hkv, G=G, BS=BS, mb=mb, k=k, sink=sink, recent=recent, flags=flags)
        oi, osc = c_api.hamming_topk(q, kc, table, lens, k, sink, recent, flags, max_blocks=mb)
        gi, gs = hamming_topk(torch.from_numpy(q.view(np.int32)).cuda(), torch.from_numpy(kc.view(np.int32)).cuda(),
                              torch.from_numpy(table).cuda(), torch.from_numpy(lens).cuda(), k, sink, recent,
                              reduce_heads=reduce_heads, return_physical=physical, distance=distance,
                              max_blocks=mb)
        assert np.array_equal(gi.cpu().numpy(), oi), what
        assert np.array_equal(gs.cpu().numpy(), osc), what
