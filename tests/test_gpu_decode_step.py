"""GPU parity of the fused decode step (encode new keys -> encode queries -> block top-k):
it must equal the separate operators, which are themselves checked against the CPU oracle,
and a HIP-graph replay of it must equal the eager result on every replay."""
import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu


def build(seed, B=4, Hq=32, Hkv=8, D=128, BS=128, nblk=6, per_head_w=True):
    from ucm_amd.sparse import HashEncoder

    rng = rng_for(seed)
    NB = B * nblk + 3
    W = torch.from_numpy(rng.standard_normal((Hkv, D, D) if per_head_w else (D, D))
                         .astype(np.float32)).to(torch.bfloat16).cuda()
    cache = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(NB, BS, Hkv, D // 32),
                                          dtype=np.int64).astype(np.int32)).cuda()
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.from_numpy(rng.integers((nblk - 1) * BS + 1, nblk * BS + 1, size=B).astype(np.int32)).cuda()
    keys = torch.from_numpy(rng.standard_normal((B, Hkv, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    qs = torch.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    # the new token of request b sits at position len-1
    pos = lens.to(torch.int64) - 1
    slots = table[torch.arange(B), (pos // BS)].to(torch.int64) * BS + pos % BS
    nw = Hkv if per_head_w else 1
    enc_k = HashEncoder(D, D, torch.bfloat16, torch.device("cuda:0"), num_weights=nw, heads_per_weight=1)
    enc_k.set_hash_weight(W)
    enc_q = HashEncoder(D, D, torch.bfloat16, torch.device("cuda:0"), num_weights=nw,
                        heads_per_weight=Hq // Hkv)
    enc_q.set_hash_weight(W)
    return W, cache, table, lens, keys, qs, slots, enc_k, enc_q


@pytest.mark.parametrize("per_head_w", [True, False])
def test_fused_step_equals_separate_operators_and_oracle(per_head_w):
    from ucm_amd.sparse import SparseDecodeStep, hamming_topk

    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(1, per_head_w=per_head_w)
    cache2 = cache.clone()
    B, Hq, Hkv, nblk, K = 4, 32, 8, 6, 3
    st = SparseDecodeStep(W, Hq, Hkv, B, nblk, K)
    idx, sc = st.step(keys, slots, qs, cache, table, lens)
    torch.cuda.synchronize()
    enc_k.compute_hash_and_cache(keys, slots, cache2, 128)
    qc = enc_q.compute_hash(qs, per_head=per_head_w).view(torch.int32)
    i2, s2 = hamming_topk(qc, cache2, table, lens, K)
    assert torch.equal(cache, cache2)
    assert torch.equal(st.q_codes, qc)
    assert torch.equal(idx, i2) and torch.equal(sc, s2)
    oi, osc = c_api.hamming_topk(qc.cpu().numpy().view(np.uint32), cache.cpu().numpy().view(np.uint32),
                                 table.cpu().numpy(), lens.cpu().numpy(), K)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(sc.cpu().numpy(), osc)


def test_bound_step_follows_tensor_contents():
    """bind() freezes the arguments, not the data: new queries in the same tensor give the new
    answer, identical to an unbound step()."""
    from ucm_amd.sparse import SparseDecodeStep

    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(3)
    B, Hq, Hkv, nblk, K = 4, 32, 8, 6, 3
    st = SparseDecodeStep(W, Hq, Hkv, B, nblk, K)
    run = st.bind(keys, slots, qs, cache, table, lens)
    i1, s1 = (t.clone() for t in run())
    e1, f1 = (t.clone() for t in st.step(keys, slots, qs, cache, table, lens))
    assert torch.equal(i1, e1) and torch.equal(s1, f1)
    qs.copy_(torch.flip(qs, dims=[0]))
    i2, s2 = (t.clone() for t in run())
    e2, f2 = (t.clone() for t in st.step(keys, slots, qs, cache, table, lens))
    assert torch.equal(i2, e2) and torch.equal(s2, f2)
    assert not torch.equal(s1, s2)


def test_step_without_new_keys_leaves_cache_untouched():
    from ucm_amd.sparse import SparseDecodeStep

    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(2)
    before = cache.clone()
    st = SparseDecodeStep(W, 32, 8, 4, 6, 2, reduce_heads=True, return_physical=True)
    idx, sc = st.step(None, None, qs, cache, table, lens)
    torch.cuda.synchronize()
    assert torch.equal(cache, before)
    qc = st.q_codes.cpu().numpy().view(np.uint32)
    oi, osc = c_api.hamming_topk(qc, cache.cpu().numpy().view(np.uint32), table.cpu().numpy(),
                                 lens.cpu().numpy(), 2, flags=c_api.F_REDUCE_HEADS | c_api.F_PHYSICAL)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(sc.cpu().numpy(), osc)


def test_graph_replays_match_eager_every_time():
    """Replay the captured step several times with eager work and synchronisations between
    the replays; inputs change between replays, so every replay must recompute."""
    from ucm_amd.sparse import SparseDecodeStep

    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(3)
    st = SparseDecodeStep(W, 32, 8, 4, 6, 3)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        st.step(keys, slots, qs, cache, table, lens)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        st.step(keys, slots, qs, cache, table, lens)
    rng = rng_for(33)
    for rep in range(4):
        # new inputs written in place (the graph reads the same buffers)
        qs.copy_(torch.from_numpy(rng.standard_normal(tuple(qs.shape)).astype(np.float32)).to(torch.bfloat16))
        keys.copy_(torch.from_numpy(rng.standard_normal(tuple(keys.shape)).astype(np.float32)).to(torch.bfloat16))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        gi, gs, gc = st.out_idx.clone(), st.out_score.clone(), cache.clone()
        ei, es = st.step(keys, slots, qs, cache, table, lens)
        torch.cuda.synchronize()
        assert torch.equal(gi, ei) and torch.equal(gs, es) and torch.equal(gc, cache)
        _ = (qs.float() @ qs.float().transpose(1, 2)).sum().item()  # unrelated eager work


def test_argument_errors():
    from ucm_amd.sparse import SparseDecodeStep

    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(4)
    st = SparseDecodeStep(W, 32, 8, 4, 6, 3)
    with pytest.raises(ValueError):
        st.step(keys, slots, qs[:, :16], cache, table, lens)
    with pytest.raises(ValueError):
        st.step(keys, slots, qs.float(), cache, table, lens)
    with pytest.raises(ValueError):
        st.step(keys, slots, qs, cache, table.to(torch.int64), lens)
    with pytest.raises(ValueError):
        SparseDecodeStep(W[:3], 32, 8, 4, 6, 3)


@pytest.mark.parametrize("Hq,T", [(64, 4), (8, 4), (1, 0), (128, 4)])
def test_fused_latent_attention_step_equals_separate_operators_and_oracle(Hq, T):
    """MLA: nope (512) + rope (64) encoders, 18-word codes, one KV head; the fused call must
    leave the same codes in the cache and return the same blocks as the separate operators;
    the replayed HIP graph of it must agree with the eager call."""
    from ucm_amd.sparse import HashEncoder, SparseDecodeStepMLA, hamming_topk

    rng = rng_for(91 + Hq)
    B, BS, nblk, K = 4, 64, 20, 5
    NB = B * nblk + 3
    dev = torch.device("cuda:0")
    en = HashEncoder(512, 512, torch.bfloat16, dev)
    er = HashEncoder(64, 64, torch.bfloat16, dev)
    cache = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(NB, BS, 18), dtype=np.int64)
                             .astype(np.int32)).cuda()
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.from_numpy(rng.integers((nblk - 1) * BS + 1, nblk * BS + 1, size=B).astype(np.int32)).cuda()
    bf = lambda shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(torch.bfloat16).cuda()
    kn, kr, qn, qr = bf((B, 512)), bf((B, 64)), bf((B, Hq, 512)), bf((B, Hq, 64))
    pos = lens.to(torch.int64) - 1
    slots = table[torch.arange(B), (pos // BS)].to(torch.int64) * BS + pos % BS
    cache2 = cache.clone()
    st = SparseDecodeStepMLA(en.hash_weights, er.hash_weights, Hq, B, nblk, K, block_size=BS,
                             sink_token=BS, recent_token=4 * BS, return_physical=True)
    args = (kn[:T] if T else None, kr[:T] if T else None, slots[:T] if T else None, qn, qr, cache, table, lens)
    idx, sc = st.step(*args)
    torch.cuda.synchronize()
    idx, sc = idx.clone(), sc.clone()
    # separate operators
    u8 = cache2.view(torch.uint8).unsqueeze(2)
    if T:
        en.compute_hash_and_cache(kn[:T, None], slots[:T], u8[..., :64], BS)
        er.compute_hash_and_cache(kr[:T, None], slots[:T], u8[..., 64:], BS)
    qc = torch.cat([en.compute_hash(qn), er.compute_hash(qr)], dim=-1).view(torch.int32)
    i2, s2 = hamming_topk(qc, cache2.unsqueeze(2), table, lens, K, BS, 4 * BS, return_physical=True)
    assert torch.equal(cache, cache2)
    assert torch.equal(st.q_codes, qc)
    assert torch.equal(idx, i2) and torch.equal(sc, s2)
    oi, osc = c_api.hamming_topk(qc.cpu().numpy().view(np.uint32),
                                 cache.cpu().numpy().view(np.uint32).reshape(NB, BS, 1, 18),
                                 table.cpu().numpy(), lens.cpu().numpy(), K, BS, 4 * BS, flags=c_api.F_PHYSICAL)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(sc.cpu().numpy(), osc)
    # graph replays (the step allocates nothing)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        st.step(*args)
    for _ in range(3):
        st.out_idx.fill_(-7)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(st.out_idx, idx) and torch.equal(st.out_score, sc)


@pytest.mark.parametrize("G", [4, 8])
def test_separate_operators_under_graph_capture(G):
    """The operators a serving engine captures one by one (encode-and-cache, query hash, block
    top-k, per-token scores) in one HIP graph: every replay, with new inputs written in place and
    eager work between the replays, must equal the eager calls and the CPU checker.  G = 8 takes
    the bit-plane path (an extra kernel and its workspace inside the graph)."""
    from ucm_amd.sparse import hamming_score, hamming_topk

    Hkv, K = 8, 3
    W, cache, table, lens, keys, qs, slots, enc_k, enc_q = build(5, Hq=Hkv * G)
    from ucm_amd.sparse import HashEncoder

    enc_q = HashEncoder(128, 128, torch.bfloat16, torch.device("cuda:0"), num_weights=Hkv, heads_per_weight=G)
    enc_q.set_hash_weight(W)
    msl = table.shape[1] * 128

    def ops():
        enc_k.compute_hash_and_cache(keys, slots, cache, 128)
        qc = enc_q.compute_hash(qs, per_head=True).view(torch.int32)
        idx, sc = hamming_topk(qc, cache, table, lens, K)
        tok = hamming_score(cache, qc[:, None], table, lens, msl, 128, 256, False, out_int32=True)
        return qc, idx, sc, tok

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        g_out = ops()
    rng = rng_for(55 + G)
    for rep in range(3):
        qs.copy_(torch.from_numpy(rng.standard_normal(tuple(qs.shape)).astype(np.float32)).to(torch.bfloat16))
        keys.copy_(torch.from_numpy(rng.standard_normal(tuple(keys.shape)).astype(np.float32)).to(torch.bfloat16))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in g_out]
        gc = cache.clone()
        want = ops()
        torch.cuda.synchronize()
        assert torch.equal(gc, cache)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        oi, osc = c_api.hamming_topk(got[0].cpu().numpy().view(np.uint32), gc.cpu().numpy().view(np.uint32),
                                     table.cpu().numpy(), lens.cpu().numpy(), K)
        assert np.array_equal(got[1].cpu().numpy(), oi) and np.array_equal(got[2].cpu().numpy(), osc)
        ot = c_api.hamming_score(got[0].cpu().numpy().view(np.uint32), gc.cpu().numpy().view(np.uint32),
                                 table.cpu().numpy(), lens.cpu().numpy(), msl, 128, 256, False)
        assert np.array_equal(got[3].cpu().numpy(), ot)
        _ = (qs.float() @ qs.float().transpose(1, 2)).sum().item()  # unrelated eager work
