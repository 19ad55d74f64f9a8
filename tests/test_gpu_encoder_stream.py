"""GPU parity of the streaming encoder kernel (the cache-build path: persistent waves, projection
matrix in registers, rows loaded straight into LDS) against the CPU oracle under the margin rule
(a bit may differ only where |projection| < 1e-2 * ||x||), and against the tiled kernel, whose
MFMA sequence it shares (identical codes expected).  The threshold hook sends small shapes to the
streaming kernel, so that the oracle stays cheap."""
import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import brute

pytestmark = pytest.mark.gpu

MARGIN_TOL = 1e-2
_DT = {torch.bfloat16: 0, torch.float16: 1}


@pytest.fixture
def stream_everything():
    from ucm_amd import _lib

    L = _lib.lib()
    L.ucm_hash_encode_set_stream_threshold(1)
    yield L
    L.ucm_hash_encode_set_stream_threshold(0)


def _encode_cache(L, x, W, slots, cache, BS, n_w, hpw):
    from ucm_amd import _lib

    T, H, K = x.shape
    N = W.shape[-1]
    _lib.check(L.ucm_hash_encode_cache(
        x.data_ptr(), _DT[x.dtype], T, H, K, x.stride(0), x.stride(1), W.data_ptr(), _DT[W.dtype], n_w, hpw, N,
        slots.data_ptr(), int(slots.dtype == torch.int64), cache.data_ptr(), cache.shape[0], BS,
        cache.stride(0), cache.stride(1), cache.stride(2), torch.cuda.current_stream().cuda_stream))


def _check_against_oracle(cache_np, x, W, slots_np, BS, hpw, rows):
    """Margin rule on the sampled token rows."""
    H = x.shape[1]
    xs = x.float().cpu().numpy()
    Ws = W.float().cpu().numpy()
    flat = cache_np.reshape(-1, H, cache_np.shape[-1])
    flips = 0
    for h in range(H):
        w = Ws[min(h // hpw, Ws.shape[0] - 1)] if hpw > 0 else Ws[0]
        ref = brute.hash_encode(xs[rows, h], w)
        got = flat[slots_np[rows], h]
        diff = np.unpackbits((got ^ ref).view(np.uint8), axis=-1, bitorder="little").astype(bool)
        marg = brute.margins(xs[rows, h], w)
        assert not np.any(diff & (marg >= MARGIN_TOL)), "bit flipped outside the margin"
        flips += int(diff.sum())
    return flips


# (seed, T, H, K, N, dtype, slot dtype, shared W)
CASES = [
    (1, 4096, 8, 128, 128, torch.bfloat16, torch.int64, False),
    (2, 4096 + 37, 8, 128, 128, torch.bfloat16, torch.int32, False),   # ragged last tile
    (3, 31, 8, 128, 128, torch.bfloat16, torch.int64, True),           # fewer rows than one tile
    (4, 3000, 4, 128, 64, torch.float16, torch.int64, False),
    (5, 5000, 2, 64, 128, torch.bfloat16, torch.int32, True),
    (6, 2048 + 1, 1, 64, 64, torch.float16, torch.int64, True),
    (7, 1500, 12, 128, 128, torch.bfloat16, torch.int64, False),       # head count that is no power of two
    (8, 70000, 8, 128, 128, torch.bfloat16, torch.int64, False),       # several tiles per wave
    # eight heads of 128-bit codes: whole cache rows stored by one wave (ring of tiles in LDS)
    (9, 70000 + 13, 8, 128, 128, torch.float16, torch.int32, False),   # ragged end after many tiles
    (10, 200000, 8, 64, 128, torch.bfloat16, torch.int64, True),       # 24 tiles per wave, ring reused 4x
    (11, 32 * 256 * 5 + 1, 8, 128, 128, torch.bfloat16, torch.int32, False),  # one tile more than the ring
    (12, 32 * 256 * 2, 8, 128, 128, torch.bfloat16, torch.int64, True),       # exactly the store delay
    # four and two heads: 64- and 32-byte rows, two and four streams per workgroup
    (13, 150000, 4, 128, 128, torch.bfloat16, torch.int64, False),
    (14, 150000 + 7, 2, 128, 128, torch.float16, torch.int32, True),
    (15, 300000, 2, 64, 128, torch.bfloat16, torch.int64, False),
]


@pytest.mark.parametrize("seed,T,H,K,N,dtype,sdt,shared", CASES)
def test_streaming_kernel_matches_oracle_and_tiled_kernel(stream_everything, seed, T, H, K, N, dtype, sdt, shared):
    L = stream_everything
    rng = rng_for(seed)
    BS = 16
    NB = -(-T // BS) + 3
    x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(dtype).cuda()
    n_w, hpw = (1, 0) if shared else (H, 1)
    W = torch.from_numpy(rng.standard_normal((n_w, K, N)).astype(np.float32)).to(dtype).cuda()
    perm = rng.permutation(NB)
    slots_np = (np.repeat(perm, BS)[:T] * BS + np.tile(np.arange(BS), NB)[:T]).astype(np.int64)
    drop = rng.choice(T, size=min(5, T), replace=False)
    slots_in = slots_np.copy()
    slots_in[drop[0]] = -1
    if len(drop) > 1:
        slots_in[drop[1]] = NB * BS + 4
    if T > 50000:  # whole tiles and runs of rows without a slot
        more = np.concatenate([np.arange(32 * 300, 32 * 302), np.arange(40001, 40040)])
        slots_in[more] = -1
        drop = np.concatenate([drop[:2], more, drop[2:]])
    slots = torch.from_numpy(slots_in).to(sdt).cuda()
    canary = 0x5A5A5A5A
    got = torch.full((NB, BS, H, N // 32), canary, dtype=torch.int32, device="cuda")
    _encode_cache(L, x, W, slots, got, BS, n_w, hpw)
    torch.cuda.synchronize()
    # the tiled kernel on the same input
    L.ucm_hash_encode_set_stream_threshold(1 << 62)
    ref = torch.full_like(got, canary)
    _encode_cache(L, x, W, slots, ref, BS, n_w, hpw)
    torch.cuda.synchronize()
    L.ucm_hash_encode_set_stream_threshold(1)
    assert torch.equal(got, ref), "streaming and tiled kernels disagree"
    g = got.cpu().numpy().view(np.uint32)
    # dropped rows and unused slots keep the canary
    flat = g.reshape(-1, H, N // 32)
    used = np.zeros(NB * BS, bool)
    keep = np.ones(T, bool)
    keep[drop[:-3] if T > 50000 else drop[:2]] = False
    used[slots_np[keep]] = True
    assert np.all(flat[~used] == canary)
    rows = np.flatnonzero(keep)
    if len(rows) > 600:
        rows = np.sort(rng.choice(rows, size=600, replace=False))
    _check_against_oracle(g, x, W, slots_np, BS, hpw, rows)


def test_streaming_kernel_dense_output(stream_everything):
    from ucm_amd import _lib

    L = stream_everything
    rng = rng_for(21)
    T, H, K, N = 2500, 8, 128, 128
    x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    W = torch.from_numpy(rng.standard_normal((H, K, N)).astype(np.float32)).to(torch.bfloat16).cuda()
    out = torch.zeros((T, H, N // 32), dtype=torch.int32, device="cuda")
    _lib.check(L.ucm_hash_encode(x.data_ptr(), 0, T, H, K, x.stride(0), x.stride(1), W.data_ptr(), 0, H, 1, N,
                                 out.data_ptr(), out.stride(0), out.stride(1),
                                 torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    o = out.cpu().numpy().view(np.uint32)
    rows = np.sort(rng.choice(T, size=500, replace=False))
    _check_against_oracle(o[:, None].reshape(T, 1, H, N // 32), x, W, np.arange(T), 1, 1, rows)


def test_streaming_kernel_dense_output_many_tiles(stream_everything):
    """Dense [T, 8, 4] output over many tiles per wave (whole 128-byte rows stored by one wave):
    identical to the tiled kernel, rows past the end untouched."""
    from ucm_amd import _lib

    L = stream_everything
    rng = rng_for(22)
    T, H, K, N = 32 * 256 * 7 + 19, 8, 128, 128
    x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    W = torch.from_numpy(rng.standard_normal((H, K, N)).astype(np.float32)).to(torch.bfloat16).cuda()
    outs = []
    for thr in (1, 1 << 62):
        L.ucm_hash_encode_set_stream_threshold(thr)
        out = torch.full((T + 64, H, N // 32), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
        _lib.check(L.ucm_hash_encode(x.data_ptr(), 0, T, H, K, x.stride(0), x.stride(1), W.data_ptr(), 0, H, 1, N,
                                     out.data_ptr(), out.stride(0), out.stride(1),
                                     torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        outs.append(out)
    L.ucm_hash_encode_set_stream_threshold(1)
    assert torch.equal(outs[0], outs[1])
    assert bool((outs[0][T:] == 0x5A5A5A5A).all())


# (seed, T, N, dtype, slot dtype, input row stride, code row words, first code word)
WIDE_CASES = [
    (31, 70000, 256, torch.bfloat16, torch.int64, 512, 8, 0),
    (32, 70000 + 13, 512, torch.bfloat16, torch.int32, 576, 18, 0),   # latent rows of 576, 18-word code rows
    (33, 40000, 512, torch.float16, torch.int64, 512, 16, 0),
    (34, 300000, 256, torch.bfloat16, torch.int32, 576, 8, 0),        # 37 tiles per workgroup, ring reused 9x
    (35, 32 * 256 * 4 + 1, 256, torch.bfloat16, torch.int64, 512, 12, 4),  # one tile more than the ring; codes at word 4
    (36, 32 * 256 * 2, 512, torch.bfloat16, torch.int64, 512, 16, 0),  # exactly two tiles per workgroup pair
    (37, 12100, 256, torch.bfloat16, torch.int32, 512, 8, 0),          # one or two tiles per workgroup: no tile loaded inside the loop
    (38, 32 * 256 * 3 - 100, 512, torch.float16, torch.int64, 576, 18, 0),  # three (a few workgroups two): the ring filled up front
    (39, 32 * 256 * 6 + 77, 256, torch.bfloat16, torch.int64, 512, 8, 0),   # six or seven: one or two steady pairs, then the tail
]


@pytest.mark.parametrize("seed,T,N,dtype,sdt,xstride,cwords,cfirst", WIDE_CASES)
def test_wide_streaming_kernel_matches_oracle_and_tiled_kernel(stream_everything, seed, T, N, dtype, sdt, xstride,
                                                               cwords, cfirst):
    """K = 512 (latent vectors): the persistent kernel that shares each row tile between the four
    waves of a workgroup, against the fp64 closed form under the margin rule and against the tiled
    kernel (same products, the k-steps added in two chains instead of one: codes may differ only where
    the projection is within rounding of zero).  Dropped slots, words of a code row that belong to
    somebody else (the rope part of a latent code) and rows past the end keep their canary."""
    from ucm_amd import _lib

    L = stream_everything
    rng = rng_for(seed)
    K, BS = 512, 64
    NB = -(-T // BS) + 3
    xfull = torch.from_numpy(rng.standard_normal((T, xstride)).astype(np.float32)).to(dtype).cuda()
    x = xfull[:, :K].unsqueeze(1)  # [T, 1, 512] with rows xstride apart
    W = torch.from_numpy(rng.standard_normal((1, K, N)).astype(np.float32)).to(dtype).cuda()
    perm = rng.permutation(NB)
    slots_np = (np.repeat(perm, BS)[:T] * BS + np.tile(np.arange(BS), NB)[:T]).astype(np.int64)
    canary = 0x5A5A5A5A
    drop = np.concatenate([rng.choice(T, size=5, replace=False), np.arange(32 * 300, 32 * 302),
                           np.arange(12001, 12040)])
    slots_in = slots_np.copy()
    slots_in[drop] = -1
    slots_in[drop[1]] = NB * BS + 4
    slots = torch.from_numpy(slots_in).to(sdt).cuda()
    outs = []
    for thr in (1, 1 << 62):
        L.ucm_hash_encode_set_stream_threshold(thr)
        cache = torch.full((NB, BS, 1, cwords), canary, dtype=torch.int32, device="cuda")
        view = cache[..., cfirst:cfirst + N // 32]
        _encode_cache(L, x, W, slots, view, BS, 1, 0)
        torch.cuda.synchronize()
        outs.append(cache)
    L.ucm_hash_encode_set_stream_threshold(1)
    got, ref = (o.cpu().numpy().view(np.uint32) for o in outs)
    codes = got[..., cfirst:cfirst + N // 32]
    # only this call's words were written
    other = np.ones(cwords, bool)
    other[cfirst:cfirst + N // 32] = False
    assert np.all(got[..., other] == canary)
    flat = codes.reshape(-1, 1, N // 32)
    keep = np.ones(T, bool)
    keep[drop] = False
    used = np.zeros(NB * BS, bool)
    used[slots_np[keep]] = True
    assert np.all(flat[~used] == canary)
    # against the tiled kernel: the same bits except within rounding of a zero projection
    diff_bits = np.unpackbits((got ^ ref).view(np.uint8)).sum()
    assert diff_bits <= max(4, T * N // 200000), f"{diff_bits} bits differ from the tiled kernel"
    rows = np.flatnonzero(keep)
    if len(rows) > 400:
        rows = np.sort(rng.choice(rows, size=400, replace=False))
    _check_against_oracle(codes, x, W, slots_np, BS, 0, rows)


@pytest.mark.parametrize("T", [50000 + 5, 3000, 33])  # 3000, 33: most workgroups have no tile at all
def test_wide_streaming_kernel_dense_output(stream_everything, T):
    from ucm_amd import _lib

    L = stream_everything
    rng = rng_for(41)
    K, N = 512, 256
    x = torch.from_numpy(rng.standard_normal((T, 1, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    W = torch.from_numpy(rng.standard_normal((1, K, N)).astype(np.float32)).to(torch.bfloat16).cuda()
    out = torch.full((T + 40, 1, N // 32), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    _lib.check(L.ucm_hash_encode(x.data_ptr(), 0, T, 1, K, x.stride(0), x.stride(1), W.data_ptr(), 0, 1, 0, N,
                                 out.data_ptr(), out.stride(0), out.stride(1),
                                 torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    o = out.cpu().numpy().view(np.uint32)
    assert np.all(o[T:] == 0x5A5A5A5A)
    rows = np.sort(rng.choice(T, size=min(400, T), replace=False))
    _check_against_oracle(o[:T].reshape(T, 1, 1, N // 32), x, W, np.arange(T), 1, 0, rows)


def test_wide_streaming_kernel_clock_probe(stream_everything):
    """The measurement aid: with a probe address set the wide kernel's first workgroup reports its
    lifetime in shader cycles and in 100 MHz ticks; the codes are the same with and without it."""
    from ucm_amd import _lib

    L = stream_everything
    rng = rng_for(43)
    T, K, N = 40000, 512, 256
    x = torch.from_numpy(rng.standard_normal((T, 1, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    W = torch.from_numpy(rng.standard_normal((1, K, N)).astype(np.float32)).to(torch.bfloat16).cuda()
    outs = []
    probe = torch.zeros(2, dtype=torch.int64, device="cuda")
    for ptr in (probe.data_ptr(), None):
        _lib.check(L.ucm_hash_encode_set_clock_probe(ptr))
        out = torch.zeros((T, 1, N // 32), dtype=torch.int32, device="cuda")
        _lib.check(L.ucm_hash_encode(x.data_ptr(), 0, T, 1, K, x.stride(0), x.stride(1), W.data_ptr(), 0, 1, 0, N,
                                     out.data_ptr(), out.stride(0), out.stride(1),
                                     torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        outs.append(out.cpu())
    cycles, ticks = (int(v) for v in probe.cpu().tolist())
    assert cycles > 10000 and ticks > 100
    ghz = cycles / (ticks * 10.0)
    assert 0.3 < ghz < 3.0, ghz
    assert torch.equal(outs[0], outs[1])
    assert L.ucm_hash_encode_set_clock_probe(probe.data_ptr() + 4) == _lib.UCM_EPARAM  # not 8-byte aligned
    _lib.check(L.ucm_hash_encode_set_clock_probe(None))


def test_no_exchange_wait_reached_its_bound():
    """The waves of the streaming kernel wait for one another with bounded polls (a launch always
    ends); after the encoder tests of this process no wait may have reached the bound."""
    from ucm_amd import _lib

    assert _lib.lib().ucm_hash_encode_stream_timeouts() == 0


def test_cache_build_size_takes_the_streaming_kernel_by_default():
    """2^20 rows (131,072 tokens x 8 KV heads of 128 -> 128 bits): the default threshold; sampled
    rows against the oracle, everything against the tiled kernel."""
    from ucm_amd import _lib

    timeouts_before = _lib.lib().ucm_hash_encode_stream_timeouts()

    L = _lib.lib()
    L.ucm_hash_encode_set_stream_threshold(0)
    rng = rng_for(33)
    T, H, K, N, BS = 131072, 8, 128, 128, 128
    NB = T // BS
    x = torch.randn((T, H, K), device="cuda", dtype=torch.bfloat16, generator=torch.Generator("cuda").manual_seed(33))
    W = torch.randn((H, K, N), device="cuda", dtype=torch.bfloat16, generator=torch.Generator("cuda").manual_seed(34))
    perm = rng.permutation(NB)
    slots_np = (np.repeat(perm, BS) * BS + np.tile(np.arange(BS), NB)).astype(np.int64)
    slots = torch.from_numpy(slots_np).cuda()
    got = torch.zeros((NB, BS, H, N // 32), dtype=torch.int32, device="cuda")
    _encode_cache(L, x, W, slots, got, BS, H, 1)
    L.ucm_hash_encode_set_stream_threshold(1 << 62)
    ref = torch.zeros_like(got)
    _encode_cache(L, x, W, slots, ref, BS, H, 1)
    L.ucm_hash_encode_set_stream_threshold(0)
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    rows = np.sort(rng.choice(T, size=400, replace=False))
    _check_against_oracle(got.cpu().numpy().view(np.uint32), x, W, slots_np, BS, 1, rows)
    assert L.ucm_hash_encode_stream_timeouts() == timeouts_before


def test_tripped_timeout_latch_surfaces_in_the_host_mirror():
    """The latch a timed-out wave sets (tripped from the host here) makes the encoder object raise
    instead of returning codes, and clearing it restores the operator."""
    from ucm_amd import _lib
    from ucm_amd.sparse import HashEncoder

    L = _lib.lib()
    enc = HashEncoder(128, 128, torch.bfloat16, torch.device("cuda"))
    x = torch.randn(64, 128, device="cuda", dtype=torch.bfloat16)
    good = enc.compute_hash(x).clone()
    assert L.ucm_hash_encode_debug_trip_stream_latch() == _lib.UCM_OK
    try:
        with pytest.raises(RuntimeError, match="gave up waiting"):
            enc.compute_hash(x)
    finally:
        assert L.ucm_hash_encode_clear_stream_timeouts() == _lib.UCM_OK
    assert torch.equal(enc.compute_hash(x), good)
