"""GPU parity: the HIP sign-hash encoder against the CPU oracle.

Tolerance rule (the only floating-point tolerance in the suite): a hash bit may differ from
the oracle only where |projection| < 1e-2 * ||x||; everywhere else it must be identical.
The oracle used for the comparison accumulates in float64.
"""
import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import brute, c_api

pytestmark = pytest.mark.gpu

MARGIN_TOL = 1e-2


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16)


def assert_codes_match(codes_u8, x32, W32):
    """codes_u8 [M, N/8] from the GPU; x32 [M,K], W32 [K,N] the exact values the GPU saw."""
    ref = brute.hash_encode(x32, W32).view(np.uint8)
    got = np.ascontiguousarray(codes_u8)
    if np.array_equal(got, ref):
        return 0
    diff_bits = np.unpackbits(got ^ ref, axis=-1, bitorder="little").astype(bool)
    marg = brute.margins(x32, W32)
    assert not np.any(diff_bits & (marg >= MARGIN_TOL)), "bit flipped outside the margin"
    return int(diff_bits.sum())


def make_encoder(K, N, dtype, W, n_w=1, hpw=1):
    from ucm_amd.sparse import HashEncoder

    enc = HashEncoder(K, N, dtype, torch.device("cuda:0"), num_weights=n_w, heads_per_weight=hpw)
    enc.set_hash_weight(W.to(dtype).cuda())
    return enc


def test_bit_and_byte_order_with_identity_weights():
    K = N = 128
    enc = make_encoder(K, N, torch.bfloat16, torch.eye(K))
    x = torch.zeros(5, K)
    x[0, 0] = 1.0
    x[1, 9] = 2.0
    x[2, 37] = 0.5
    x[2, 3] = -1.0
    x[3, 127] = 3.0
    x[4, :] = -1.0
    codes = enc.compute_hash(x.to(torch.bfloat16).cuda()).cpu().numpy()
    words = np.ascontiguousarray(codes).view("<u4")
    assert words[0].tolist() == [1, 0, 0, 0]
    assert words[1].tolist() == [1 << 9, 0, 0, 0]
    assert words[2].tolist() == [0, 1 << 5, 0, 0]
    assert words[3].tolist() == [0, 0, 0, 1 << 31]
    assert words[4].tolist() == [0, 0, 0, 0]
    assert codes[1, 1] == 2  # byte 1, bit 1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K,N", [(1, 128, 128), (33, 128, 128), (300, 128, 128),
                                   (70, 64, 64), (40, 256, 128), (50, 512, 256), (17, 128, 96)])
def test_compute_hash_matches_oracle(dtype, M, K, N):
    rng = rng_for(1000 + M + K + N)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    W = torch.from_numpy(rng.standard_normal((K, N)).astype(np.float32)).to(dtype)
    enc = make_encoder(K, N, dtype, W)
    codes = enc.compute_hash(x.cuda())
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == (M, N // 8)
    assert_codes_match(codes.cpu().numpy(), x.float().numpy(), W.float().numpy())


def test_leading_dims_and_negation():
    rng = rng_for(7)
    x = bf16_round(rng.standard_normal((3, 5, 128)))
    W = bf16_round(rng.standard_normal((128, 128)))
    enc = make_encoder(128, 128, torch.bfloat16, W)
    c = enc.compute_hash(x.cuda())
    assert tuple(c.shape) == (3, 5, 16)
    cn = enc.compute_hash((-x).cuda())
    assert torch.equal(cn, ~c)  # no projection is exactly zero for Gaussian data


def test_zero_and_nan_rows_give_zero_bits():
    enc = make_encoder(128, 128, torch.bfloat16, torch.eye(128))
    x = torch.zeros(2, 128)
    x[1, 2] = float("nan")
    x[1, 5] = 1.0
    c = enc.compute_hash(x.to(torch.bfloat16).cuda()).cpu().numpy()
    assert not c.any()


def test_per_head_weights_gqa_queries():
    """BASELINE.json config 2 query side: 32 q heads, one projection per KV head (group of 4)."""
    rng = rng_for(8)
    B, Hq, Hkv, K, N = 6, 32, 8, 128, 128
    x = bf16_round(rng.standard_normal((B, Hq, K)))
    W = bf16_round(rng.standard_normal((Hkv, K, N)))
    enc = make_encoder(K, N, torch.bfloat16, W, n_w=Hkv, hpw=Hq // Hkv)
    c = enc.compute_hash(x.cuda(), per_head=True).cpu().numpy()
    assert c.shape == (B, Hq, N // 8)
    for h in range(Hq):
        assert_codes_match(c[:, h], x[:, h].float().numpy(), W[h // 4].float().numpy())


@pytest.mark.parametrize("B,H,K,N,n_w", [
    (16, 64, 512, 512, 1),   # the latent-attention step's queries: 32 tiles of (token, head) pairs instead of 64 half-empty ones
    (3, 5, 128, 128, 1),     # 15 pairs: one partial tile
    (33, 3, 64, 64, 1),      # 99 pairs in 4 tiles against 2 x 3 by head
    (7, 6, 256, 256, 1),
    (40, 4, 128, 128, 1),    # 2 x 4 tiles by head, 5 by pair
    (7, 6, 128, 128, 2),     # two projections (3 heads each): tiles stay with one head
])
def test_few_tokens_many_heads_one_projection(B, H, K, N, n_w):
    """Rows of the small-row kernel's tiles are (token, head) pairs when one projection serves every
    head and that needs fewer tiles; the codes, and where they go (dense and through a slot mapping),
    are the same as head by head."""
    rng = rng_for(80 + B + H)
    x = bf16_round(rng.standard_normal((B, H, K)))
    W = bf16_round(rng.standard_normal((n_w, K, N)))
    hpw = H // n_w
    enc = make_encoder(K, N, torch.bfloat16, W, n_w=n_w, hpw=hpw)
    c = enc.compute_hash(x.cuda(), per_head=True).cpu().numpy()
    assert c.shape == (B, H, N // 8)
    for h in range(H):
        assert_codes_match(c[:, h], x[:, h].float().numpy(), W[h // hpw].float().numpy())
    # the same rows through the paged store, two dropped
    NB, BS = 5, 16
    slots = rng.permutation(NB * BS)[:B].astype(np.int64)
    slots[0] = -1
    if B > 2:
        slots[2] = NB * BS + 3
    cache = torch.full((NB, BS, H, N // 8), 0xAB, dtype=torch.uint8, device="cuda")
    enc.compute_hash_and_cache(x.cuda(), torch.from_numpy(slots).cuda(), cache, block_size=BS)
    expect = np.full((NB, BS, H, N // 32), 0xABABABAB, np.uint32)
    c_api.code_scatter(np.ascontiguousarray(c).view(np.uint32), slots, expect, BS)
    assert np.array_equal(cache.cpu().numpy().view(np.uint32), expect)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("slot_dtype", [torch.int32, torch.int64])
def test_compute_hash_and_cache(dtype, slot_dtype):
    rng = rng_for(9)
    T, H, K, N, NB, BS = 200, 8, 128, 128, 6, 128
    x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(dtype)
    W = torch.from_numpy(rng.standard_normal((H, K, N)).astype(np.float32)).to(dtype)
    slots = rng.permutation(NB * BS)[:T].astype(np.int64)
    slots[5] = -1
    slots[17] = NB * BS          # first slot past the cache
    slots[40] = NB * BS + 1000
    enc = make_encoder(K, N, dtype, W, n_w=H, hpw=1)
    cache = torch.full((NB, BS, H, N // 8), 0xAB, dtype=torch.uint8, device="cuda")
    out = enc.compute_hash_and_cache(x.cuda(), torch.from_numpy(slots).to(slot_dtype).cuda(),
                                     cache, block_size=BS)
    assert out is cache
    got = cache.cpu().numpy()
    # fused write == separate encode + the oracle's scatter (hash_encoder.py:136-195)
    codes = enc.compute_hash(x.cuda(), per_head=True).cpu().numpy()  # [T,H,16]
    expect = np.full((NB, BS, H, N // 32), 0xABABABAB, np.uint32)
    c_api.code_scatter(np.ascontiguousarray(codes).view(np.uint32), slots, expect, BS)
    assert np.array_equal(got.view(np.uint32), expect)
    for h in range(H):
        assert_codes_match(codes[:, h], x[:, h].float().numpy(), W[h].float().numpy())


# Row counts above 256 per head take the tiled MFMA kernel; the shapes below reach each of its
# compile-time variants: column tiles per group 4/2/1, unrolled and run-time group counts,
# the pipelined path (K <= 128) and the line-by-line path (K >= 256), partial last tiles and
# workgroups whose run of tiles ends past the tensor.
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N", [(257, 128, 128), (515, 128, 128), (1000, 128, 256), (4100, 128, 128),
                                   (700, 128, 512), (300, 128, 192), (300, 128, 96), (640, 128, 64),
                                   (385, 128, 32), (513, 64, 64), (900, 64, 128), (300, 64, 32),
                                   (600, 256, 128), (300, 512, 256), (2049, 512, 128)])
def test_tiled_kernel_shapes(dtype, M, K, N):
    rng = rng_for(2000 + M + K + N)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    W = torch.from_numpy(rng.standard_normal((K, N)).astype(np.float32)).to(dtype)
    enc = make_encoder(K, N, dtype, W)
    codes = enc.compute_hash(x.cuda())
    assert tuple(codes.shape) == (M, N // 8)
    assert_codes_match(codes.cpu().numpy(), x.float().numpy(), W.float().numpy())


@pytest.mark.parametrize("slot_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("T,H,BS", [(700, 8, 128), (1029, 4, 48), (300, 2, 16)])
def test_tiled_kernel_paged_store(slot_dtype, T, H, BS):
    """Fused cache write of the tiled kernel: permuted and invalid slots, a block size that is
    not a power of two, head-interleaved input rows, cells outside the slots untouched."""
    rng = rng_for(12 + T)
    K = N = 128
    NB = (T + BS - 1) // BS + 3
    x = bf16_round(rng.standard_normal((T, H, K)))
    W = bf16_round(rng.standard_normal((H, K, N)))
    slots = rng.permutation(NB * BS)[:T].astype(np.int64)
    slots[3] = -1
    slots[T // 2] = NB * BS
    slots[T - 1] = NB * BS + 77
    enc = make_encoder(K, N, torch.bfloat16, W, n_w=H, hpw=1)
    cache = torch.full((NB, BS, H, N // 8), 0xAB, dtype=torch.uint8, device="cuda")
    enc.compute_hash_and_cache(x.cuda(), torch.from_numpy(slots).to(slot_dtype).cuda(), cache,
                               block_size=BS)
    codes = np.stack([brute.hash_encode(x[:, h].float().numpy(), W[h].float().numpy())
                      for h in range(H)], axis=1)  # [T,H,4] uint32
    expect = np.full((NB, BS, H, N // 32), 0xABABABAB, np.uint32)
    c_api.code_scatter(np.ascontiguousarray(codes), slots, expect, BS)
    got = cache.cpu().numpy().view(np.uint32)
    if not np.array_equal(got, expect):
        # differences may only be margin bits of rows that were written
        gpu_codes = enc.compute_hash(x.cuda(), per_head=True).cpu().numpy()
        for h in range(H):
            assert_codes_match(gpu_codes[:, h], x[:, h].float().numpy(), W[h].float().numpy())
        expect2 = np.full((NB, BS, H, N // 32), 0xABABABAB, np.uint32)
        c_api.code_scatter(np.ascontiguousarray(gpu_codes).view(np.uint32), slots, expect2, BS)
        assert np.array_equal(got, expect2)


def test_tiled_kernel_strided_rows_and_dense_heads():
    """Rows that are a slice of a wider tensor (row pitch 3*K) and a dense per-head output."""
    rng = rng_for(13)
    T, H, K, N = 520, 3, 128, 128
    wide = bf16_round(rng.standard_normal((T, H, 3 * K))).cuda()
    x = wide[:, :, K:2 * K]
    W = bf16_round(rng.standard_normal((K, N)))
    enc = make_encoder(K, N, torch.bfloat16, W)
    c = enc.compute_hash(x, per_head=True).cpu().numpy()  # keeps the row pitch; one matrix
    assert c.shape == (T, H, N // 8)
    xs = x.float().cpu().numpy()
    for h in range(H):
        assert_codes_match(c[:, h], xs[:, h], W.float().numpy())


@pytest.mark.parametrize("dtype,BS,H,n_blocks,n_tokens,per_head", [
    (torch.bfloat16, 128, 8, 9, 1100, True),    # tiled kernel, partial last block
    (torch.float16, 128, 2, 40, 5120, False),   # several workgroups per head
    (torch.bfloat16, 64, 4, 3, 130, False),     # few rows: latency kernel
    (torch.bfloat16, 32, 4, 20, 640, True),     # a wave per block
    (torch.bfloat16, 48, 2, 12, 570, False),    # block size not a multiple of 32: FMA kernel
    (torch.float32, 16, 2, 5, 77, False),       # fp32: FMA kernel
])
def test_rehash_from_paged_cache(dtype, BS, H, n_blocks, n_tokens, per_head):
    """Prefix-cache rehash against the CPU checker and against the reference's own recipe run
    on the GPU (gather the blocks, then compute_hash_and_cache with the prefix slot mapping)."""
    rng = rng_for(300 + BS + n_blocks)
    K = N = 128
    NBk, NB = n_blocks + 6, n_blocks + 4
    kc = torch.from_numpy(rng.standard_normal((NBk, BS, H, K)).astype(np.float32)).to(dtype)
    W = torch.from_numpy(rng.standard_normal((H if per_head else 1, K, N)).astype(np.float32)).to(dtype)
    ids = rng.permutation(NB)[:n_blocks].astype(np.int32)
    if n_blocks >= 5:
        ids[1] = -1            # unusable entries drop their tokens
        ids[3] = NB + 1        # valid in the KV cache, outside the code cache
    enc = make_encoder(K, N, dtype, W if per_head else W[0], n_w=H if per_head else 1, hpw=1)
    cache = torch.full((NB, BS, H, N // 8), 0xAB, dtype=torch.uint8, device="cuda")
    out = enc.compute_hash_from_paged_cache(kc.cuda(), torch.from_numpy(ids).cuda(), n_tokens, cache,
                                            block_size=BS)
    assert out is cache
    got = cache.cpu().numpy().view(np.uint32)

    # the reference's recipe on the GPU: gather, slot mapping, fused encode + store
    cache2 = torch.full_like(cache, 0xAB)
    tok = np.arange(n_tokens)
    slots = ids[tok // BS].astype(np.int64) * BS + tok % BS
    slots[(ids[tok // BS] < 0) | (ids[tok // BS] >= NB)] = -1
    gathered = kc.cuda()[torch.from_numpy(np.clip(ids, 0, NBk - 1)).long().cuda()].reshape(-1, H, K)[:n_tokens]
    enc.compute_hash_and_cache(gathered.contiguous(), torch.from_numpy(slots).cuda(), cache2, block_size=BS)
    assert torch.equal(cache, cache2)

    # CPU checker (bits may differ only inside the margin)
    expect = np.full((NB, BS, H, N // 32), 0xABABABAB, np.uint32)
    c_api.hash_encode_paged(kc.float().numpy(), ids, n_tokens, W.float().numpy(),
                            1 if per_head else 0, expect)
    if not np.array_equal(got, expect):
        kcn, Wn = kc.float().numpy(), W.float().numpy()
        for i in range(n_tokens):
            b = int(ids[i // BS])
            if b < 0 or b >= NB:
                continue
            for h in range(H):
                assert_codes_match(got[b, i % BS, h:h + 1].view(np.uint8),
                                   kcn[b, i % BS, h:h + 1], Wn[h if per_head else 0])
    # cells of skipped and unlisted blocks stay untouched
    listed = {int(b) for b in ids if 0 <= b < NB}
    for b in range(NB):
        if b not in listed:
            assert (got[b] == 0xABABABAB).all()


def test_rehash_argument_errors():
    enc = make_encoder(128, 128, torch.bfloat16, torch.eye(128))
    kc = torch.zeros((4, 64, 2, 128), dtype=torch.bfloat16, device="cuda")
    cache = torch.zeros((4, 64, 2, 16), dtype=torch.uint8, device="cuda")
    ids = torch.tensor([0, 1], dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        enc.compute_hash_from_paged_cache(kc, ids, 129, cache, block_size=64)   # > 2 blocks
    with pytest.raises(ValueError):
        enc.compute_hash_from_paged_cache(kc, ids.long(), 10, cache, block_size=64)
    with pytest.raises(ValueError):
        enc.compute_hash_from_paged_cache(kc, ids, 10, cache, block_size=128)
    with pytest.raises(ValueError):
        enc.compute_hash_from_paged_cache(kc.float(), ids, 10, cache, block_size=64)
    assert enc.compute_hash_from_paged_cache(kc, ids, 0, cache, block_size=64) is cache


def test_cache_as_bf16_view_and_shared_weight():
    """The plugin allocates the code cache as bfloat16 [NB,BS,H,hash_numbers/2]
    (hash_encoder.py:509-546) and uses one projection for all heads."""
    rng = rng_for(10)
    T, H, K, N, NB, BS = 64, 4, 128, 128, 2, 64
    x = bf16_round(rng.standard_normal((T, H, K)))
    W = bf16_round(rng.standard_normal((K, N)))
    enc = make_encoder(K, N, torch.bfloat16, W)
    cache = torch.zeros((NB, BS, H, N // 16), dtype=torch.bfloat16, device="cuda")
    slots = torch.arange(T, dtype=torch.int64, device="cuda") + 10
    enc.compute_hash_and_cache(x.cuda(), slots, cache, block_size=BS)
    got = cache.view(torch.uint8).cpu().numpy().reshape(NB * BS, H, N // 8)
    for h in range(H):
        assert_codes_match(got[10:10 + T, h], x[:, h].float().numpy(), W.float().numpy())
    assert not got[:10].any() and not got[10 + T:].any()


def test_reshape_and_cache_head_major_shape_of_the_reference_fixture():
    """Shapes of ucm/sparse/test/gsa/pt/npu_reshape_and_cache_bnsd_tensor.pt (that file holds
    inputs only): 1 token, 2 heads, 16-byte codes, slot 22552, head-major cache
    [402, 2, 128, 16].  Data here is synthetic."""
    from ucm_amd.sparse.hash_encoder import reshape_and_cache_khash

    rng = rng_for(11)
    codes = torch.from_numpy(rng.integers(0, 256, size=(1, 2, 16), dtype=np.uint8)).cuda()
    cache_hm = torch.zeros((402, 2, 128, 16), dtype=torch.uint8, device="cuda")
    slot = torch.tensor([22552], dtype=torch.int32, device="cuda")
    # token-major view [NB, BS, H, W] of the head-major storage
    reshape_and_cache_khash(codes, slot, cache_hm.permute(0, 2, 1, 3), block_size=128)
    got = cache_hm.cpu().numpy()
    assert np.array_equal(got[176, :, 24, :], codes[0].cpu().numpy())
    got[176, :, 24, :] = 0
    assert not got.any()


def test_argument_errors_match_the_reference_behaviour():
    from ucm_amd.sparse import HashEncoder

    with pytest.raises(ValueError):
        HashEncoder(128, 100, torch.bfloat16, torch.device("cuda:0"))
    enc = HashEncoder(128, 128, torch.bfloat16, torch.device("cuda:0"))
    with pytest.raises(ValueError):
        enc.compute_hash(torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        enc.compute_hash(torch.zeros(4, 128, dtype=torch.bfloat16))  # wrong device
    with pytest.raises(ValueError):
        enc.set_hash_weight(torch.zeros(128, 64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        enc.set_hash_weight(torch.zeros(128, 128, dtype=torch.float32, device="cuda"))
    cache = torch.zeros((2, 64, 4, 16), dtype=torch.uint8, device="cuda")
    x = torch.zeros(3, 4, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        enc.compute_hash_and_cache(x, torch.zeros(2, dtype=torch.int64, device="cuda"), cache, 64)
    with pytest.raises(ValueError):
        enc.compute_hash_and_cache(x, torch.zeros(3, dtype=torch.int64, device="cuda"), cache, 128)
    # Haar-orthogonal default weights: W^T W = I
    w = enc.hash_weights.float()
    assert torch.allclose(w.T @ w, torch.eye(128, device="cuda"), atol=5e-2)


def test_unpack_hash_roundtrip():
    enc = make_encoder(128, 128, torch.bfloat16, torch.eye(128))
    x = torch.zeros(2, 128)
    x[0, 3] = 1.0
    x[1, 100] = 1.0
    c = enc.compute_hash(x.to(torch.bfloat16).cuda())
    pm = enc._unpack_hash(c).cpu()
    assert pm[0, 3] == 1 and pm[1, 100] == 1 and pm.sum() == 2 - (256 - 2)
