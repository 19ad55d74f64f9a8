"""GPU tests of the reference-shaped surfaces around the operators: the retrieval worker API,
the sparse plugin hooks and the KV store interface."""
import os
import types

import numpy as np
import pytest
import torch

from helpers import assert_topk_matches_unordered_ties, rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "hash_retrieval_ref.npz")


@pytest.mark.parametrize("case,k", [("ragged", 5), ("ragged", 10), ("tail", 12), ("zero", 3)])
def test_retrieval_worker_matches_the_reference_backend_outputs(case, k):
    """Same submit/wait/get_result calls as the reference's worker, compared with the outputs the
    reference's CPU backend produced for these inputs (golden fixture) and with the oracle."""
    from ucm_amd.sparse.retrieval_worker import HashRetrievalWorker, HashRetrievalWorkerBackend

    gold = np.load(GOLD)
    data, query = gold[f"{case}_data"], gold[f"{case}_query"]
    if case == "ragged":
        indexes = gold["ragged_indexes"]
        ref_i, ref_d = gold[f"ragged_idx_k{k}"], gold[f"ragged_dist_k{k}"]
    else:
        indexes = np.tile(np.arange(data.shape[0], dtype=np.int32), (query.shape[0], 1))
        ref_i, ref_d = gold[f"{case}_idx"], gold[f"{case}_dist"]
    worker = HashRetrievalWorker(HashRetrievalWorkerBackend(data, {0: [0]}))
    rid = worker.submit(torch.from_numpy(query), k, indexes)
    worker.wait(rid)
    assert worker.poll(rid)
    res = worker.get_result(rid)
    with pytest.raises(RuntimeError):
        worker.get_result(rid)  # consumed once
    oi, od, on = c_api.hash_retrieval(data, query, indexes, k)
    for r in range(query.shape[0]):
        kk = int(on[r])
        assert np.array_equal(res["indices"][r, :kk], oi[r, :kk])  # same tie rule as the oracle
        assert np.array_equal(res["scores"][r, :kk], od[r, :kk])
        assert np.array_equal(res["scores"][r, :kk], ref_d[r, :kk])
        fi, fd, fn = c_api.hash_retrieval(data, query[r:r + 1], indexes[r:r + 1], indexes.shape[1])
        score_of = {int(i): int(s) for i, s in zip(fi[0, : fn[0]], fd[0, : fn[0]])}
        assert_topk_matches_unordered_ties(res["indices"][r, :kk], res["scores"][r, :kk],
                                           ref_i[r, :kk], ref_d[r, :kk], all_scores=score_of)


def test_retrieval_worker_errors():
    from ucm_amd.sparse.retrieval_worker import HashRetrievalWorkerBackend

    be = HashRetrievalWorkerBackend(np.zeros((4, 8, 16), np.uint8))
    with pytest.raises(RuntimeError):
        be.submit(np.zeros((1, 8), np.uint8), 2, np.zeros((1, 4), np.int32))
    with pytest.raises(RuntimeError):
        be.submit(np.zeros((2, 16), np.uint8), 2, np.zeros((1, 4), np.int32))
    with pytest.raises(RuntimeError):
        be.wait(99)
    with pytest.raises(RuntimeError):
        be.get_result(99)


def test_plugin_hooks_swap_and_restore_the_block_table():
    from ucm_amd.sparse.base import UcmSparseFactory, UcmSparseRole

    B, Hq, Hkv, D, BS, nblk, topk_tok = 3, 32, 8, 128, 128, 24, 1024
    cfg = {"ucm_sparse_config": {"GSAOnDevice": {
        "num_q_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "block_size": BS,
        "vllm_hash_attention_topk": topk_tok, "vllm_hash_attention_rollback_layers": [0],
        "seed": 5}}}
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    rng = rng_for(77)
    NB = B * nblk + 2
    k_hash = torch.zeros((NB, BS, Hkv, D // 8), dtype=torch.uint8, device="cuda")
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.tensor([nblk * BS, nblk * BS - 300, 5 * BS + 1], dtype=torch.int32, device="cuda")
    # prefill: hash every token's key into the code cache through the hook
    for b in range(B):
        L = int(lens[b])
        keys = torch.from_numpy(rng.standard_normal((L, Hkv * D)).astype(np.float32)).to(torch.bfloat16).cuda()
        pos = torch.arange(L, device="cuda")
        slots = table[b, pos // BS].long() * BS + pos % BS
        meta = types.SimpleNamespace(slot_mapping=slots, block_table=table[b:b + 1], seq_lens=lens[b:b + 1])
        ctx = types.SimpleNamespace(attn_metadata={"model.layers.1.self_attn.attn": meta})
        plugin.attention_begin(None, keys, None, "model.layers.1.self_attn.attn", ctx,
                               phase="prefill", k_hash=k_hash)
    assert int((k_hash != 0).sum()) > 0
    # decode step on a normal layer
    q = torch.from_numpy(rng.standard_normal((B, Hq * D)).astype(np.float32)).to(torch.bfloat16).cuda()
    newk = torch.from_numpy(rng.standard_normal((B, Hkv * D)).astype(np.float32)).to(torch.bfloat16).cuda()
    pos = lens.long() - 1
    slots = table[torch.arange(B), pos // BS].long() * BS + pos % BS
    meta = types.SimpleNamespace(slot_mapping=slots, block_table=table.clone(), seq_lens=lens.clone())
    ctx = types.SimpleNamespace(attn_metadata={"model.layers.1.self_attn.attn": meta})
    plugin.attention_begin(q, newk, None, "model.layers.1.self_attn.attn", ctx, phase="decode",
                           k_hash=k_hash)
    kblk = topk_tok // BS
    # expected: oracle on the codes now in the cache, group-mean query code per KV head
    qc = plugin.hash_code(q.view(B, Hq, D)).cpu().numpy().view(np.uint32)
    codes = k_hash.cpu().numpy().view(np.uint32).reshape(NB, BS, Hkv, D // 32)
    oi, _ = c_api.hamming_topk(qc, codes, table.cpu().numpy(), lens.cpu().numpy(), kblk, BS, 4 * BS,
                               flags=c_api.F_REDUCE_HEADS | c_api.F_PHYSICAL)
    got = meta.block_table.cpu().numpy()
    assert np.array_equal(got[:, :kblk], np.maximum(oi[:, 0], 0))
    assert not got[:, kblk:].any()
    assert np.array_equal(meta.seq_lens.cpu().numpy(), c_api.update_seq_lens(lens.cpu().numpy(), topk_tok, BS))
    plugin.attention_finished(q, newk, None, None, "model.layers.1.self_attn.attn", ctx, phase="decode")
    assert torch.equal(meta.block_table, table) and torch.equal(meta.seq_lens, lens)
    # a rollback layer keeps the full table
    meta0 = types.SimpleNamespace(slot_mapping=slots, block_table=table.clone(), seq_lens=lens.clone())
    ctx0 = types.SimpleNamespace(attn_metadata=meta0)
    plugin.attention_begin(q, newk, None, "model.layers.0.self_attn.attn", ctx0, phase="decode",
                           k_hash=k_hash)
    assert torch.equal(meta0.block_table, table)


@pytest.mark.parametrize("threshold", [0, 2000])
def test_plugin_single_call_decode_equals_separate_operators_and_oracle(threshold):
    """attention_begin at decode as ONE native call (ucm_gsa_decode_step) against the same hook
    running the separate operators (encode-and-cache, mean-query hash, top-k, torch table swap)
    and against the CPU checker: identical code cache, replacement table and lengths.  Lengths
    include a request shorter than the top-k budget, one shorter than the threshold and a ragged
    last block."""
    from ucm_amd.sparse.base import UcmSparseFactory, UcmSparseRole

    B, Hq, Hkv, D, BS, nblk, topk_tok = 5, 32, 8, 128, 128, 40, 2048
    name = "model.layers.3.self_attn.attn"
    rng = rng_for(91)
    NB = B * nblk + 3
    base_codes = torch.from_numpy(rng.integers(0, 256, size=(NB, BS, Hkv, D // 8), dtype=np.uint8)).cuda()
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.tensor([nblk * BS, nblk * BS - 300, 9 * BS + 1, 1500, 17 * BS], dtype=torch.int32, device="cuda")
    q = torch.from_numpy(rng.standard_normal((B, Hq * D)).astype(np.float32)).to(torch.bfloat16).cuda()
    newk = torch.from_numpy(rng.standard_normal((B, Hkv * D)).astype(np.float32)).to(torch.bfloat16).cuda()
    pos = lens.long() - 1
    slots = table[torch.arange(B), pos // BS].long() * BS + pos % BS
    results = []
    for fused in (True, False):
        cfg = {"ucm_sparse_config": {"GSAOnDevice": {
            "num_q_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "block_size": BS,
            "vllm_hash_attention_topk": topk_tok, "gpu_seq_len_threshold": threshold,
            "fused_decode": fused, "seed": 11}}}
        plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
        k_hash = base_codes.clone()
        meta = types.SimpleNamespace(slot_mapping=slots, block_table=table.clone(), seq_lens=lens.clone())
        ctx = types.SimpleNamespace(attn_metadata={name: meta})
        for _ in range(2):  # twice: the step's buffers are reused
            plugin.attention_begin(q, newk, None, name, ctx, phase="decode", k_hash=k_hash)
            torch.cuda.synchronize()
            out = (k_hash.clone(), meta.block_table.clone(), meta.seq_lens.clone())
            plugin.attention_finished(q, newk, None, None, name, ctx, phase="decode")
            assert torch.equal(meta.block_table, table) and torch.equal(meta.seq_lens, lens)
        results.append((plugin, out))
    (pf, (kh_f, bt_f, sl_f)), (ps, (kh_s, bt_s, sl_s)) = results
    assert torch.equal(pf.hash_encoder.hash_weights, ps.hash_encoder.hash_weights)
    assert torch.equal(kh_f, kh_s), "code cache differs between the single call and the separate operators"
    assert torch.equal(bt_f, bt_s) and torch.equal(sl_f, sl_s)
    # the query codes of the single call are the codes of torch's group mean
    step = next(iter(pf._fused_steps.values()))
    qc_sep = ps.hash_code(q.view(B, Hq, D)).view(torch.int32)
    assert torch.equal(step.q_codes, qc_sep)
    # and the CPU checker on the codes now in the cache
    kblk = topk_tok // BS
    oi, _ = c_api.hamming_topk(step.q_codes.cpu().numpy().view(np.uint32),
                               kh_f.cpu().numpy().view(np.uint32).reshape(NB, BS, Hkv, D // 32),
                               table.cpu().numpy(), lens.cpu().numpy(), kblk, BS, 4 * BS,
                               flags=c_api.F_REDUCE_HEADS | c_api.F_PHYSICAL)
    exp_t = np.zeros((B, nblk), np.int32)
    exp_t[:, :kblk] = np.maximum(oi[:, 0], 0)
    exp_l = c_api.update_seq_lens(lens.cpu().numpy(), topk_tok, BS)
    if threshold:
        short = lens.cpu().numpy() < threshold
        exp_t[short] = table.cpu().numpy()[short]
        exp_l[short] = lens.cpu().numpy()[short]
        assert short.any() and not short.all()
    assert np.array_equal(bt_f.cpu().numpy(), exp_t)
    assert np.array_equal(sl_f.cpu().numpy(), exp_l)


def test_single_call_decode_step_in_a_hip_graph():
    """GSADecodeStep allocates nothing: captured once, replayed with changing inputs, every replay
    checked against an eager call."""
    from ucm_amd.sparse import GSADecodeStep

    B, Hq, Hkv, D, BS, nblk, topk_tok = 4, 32, 8, 128, 128, 32, 1024
    rng = rng_for(92)
    NB = B * nblk
    W = torch.from_numpy(rng.standard_normal((D, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    cache = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(NB, BS, Hkv, D // 32), dtype=np.int64)
                             .astype(np.int32)).cuda()
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.full((B,), nblk * BS, dtype=torch.int32, device="cuda")
    q = torch.empty((B, Hq, D), dtype=torch.bfloat16, device="cuda")
    newk = torch.empty((B, Hkv, D), dtype=torch.bfloat16, device="cuda")
    slots = (table[:, -1].long() * BS + BS - 1)
    step = GSADecodeStep(W, Hq, Hkv, B, nblk, topk_tok, block_size=BS)
    eager = GSADecodeStep(W, Hq, Hkv, B, nblk, topk_tok, block_size=BS)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        q.normal_(); newk.normal_()
        step.step(newk, slots, q, cache, table, lens)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step.step(newk, slots, q, cache, table, lens)
    for it in range(4):
        q.normal_(); newk.normal_()
        lens[it % B] -= 37 * (it + 1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = (step.new_table.clone(), step.new_lens.clone(), step.q_codes.clone())
        eager.step(newk, slots, q, cache, table, lens)
        torch.cuda.synchronize()
        assert torch.equal(got[0], eager.new_table) and torch.equal(got[1], eager.new_lens)
        assert torch.equal(got[2], eager.q_codes)


def test_plugin_rehashes_a_prefix_cache_hit_from_the_key_cache():
    """Two requests whose prompt prefixes were loaded from the store into the paged KV cache:
    the hook must produce, for the prefix tokens, the codes a full prefill of the same keys
    would have produced (gsa_on_device.py:574-588), next to the codes of the new tokens."""
    from ucm_amd.sparse.base import UcmSparseFactory, UcmSparseRole

    Hq, Hkv, D, BS = 32, 8, 128, 64
    cfg = {"ucm_sparse_config": {"GSAOnDevice": {
        "num_q_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "block_size": BS, "seed": 6}}}
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    rng = rng_for(78)
    NB = 40
    name = "model.layers.1.self_attn.attn"
    k_cache = torch.from_numpy(rng.standard_normal((NB, BS, Hkv, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    rows = torch.from_numpy(rng.permutation(NB)[:24].astype(np.int32).reshape(2, 12)).cuda()
    prompts, qlens = [9 * BS + 17, 6 * BS], [BS + 17, 2 * BS]   # prefixes of 8 and 4 blocks
    # new tokens of the step (their keys also sit in the KV cache, as after the cache write)
    pos = [torch.arange(p - q, p, device="cuda") for p, q in zip(prompts, qlens)]
    slots = torch.cat([rows[b, ps // BS].long() * BS + ps % BS for b, ps in enumerate(pos)])
    keys = k_cache.view(NB * BS, Hkv * D)[slots]
    k_hash = torch.zeros((NB, BS, Hkv, D // 8), dtype=torch.uint8, device="cuda")
    plugin.set_prefix_cache_hits([(rows[0], prompts[0], qlens[0]), (rows[1], prompts[1], qlens[1])])
    assert plugin.has_pc_hit and plugin.prefix_block_ids.numel() == 12
    assert plugin.prefix_slot_mapping.numel() == 8 * BS + 4 * BS
    meta = types.SimpleNamespace(slot_mapping=slots, block_table=rows, seq_lens=None)
    layer = types.SimpleNamespace(kv_cache=[(k_cache, None)])
    ctx = types.SimpleNamespace(attn_metadata={name: meta}, no_compile_layers={name: layer}, virtual_engine=0)
    plugin.attention_begin(None, keys, None, name, ctx, phase="prefill", k_hash=k_hash)
    # expected: every prompt token's key hashed at its slot
    expect = torch.zeros_like(k_hash)
    allpos = [torch.arange(p, device="cuda") for p in prompts]
    allslots = torch.cat([rows[b, ps // BS].long() * BS + ps % BS for b, ps in enumerate(allpos)])
    plugin.hash_encoder.compute_hash_and_cache(
        k_cache.view(NB * BS, Hkv, D)[allslots], allslots, expect, block_size=BS)
    assert torch.equal(k_hash, expect)
    # the slot mapping the mirror reports equals the reference's formula
    assert torch.equal(plugin.prefix_slot_mapping[: 8 * BS], allslots[: 8 * BS])


def test_plugin_latent_attention_mode():
    """MLA: nope (512) and rope (64) parts hashed by two encoders into 18-word codes
    (gsa_on_device.py:210-232,426-455), decode query heads averaged down by
    reduction_head_num and compared as 8 query codes against the one latent head (:667-709)."""
    from ucm_amd.sparse.base import UcmSparseFactory, UcmSparseRole

    B, Hq, BS, nblk, topk_tok, red = 3, 16, 64, 20, 512, 2
    cfg = {"ucm_sparse_config": {"GSAOnDevice": {
        "num_q_heads": Hq, "num_kv_heads": 1, "head_dim": 576, "block_size": BS, "is_mla": True,
        "kv_lora_rank": 512, "qk_rope_head_dim": 64, "vllm_hash_attention_reduction_head_num": red,
        "vllm_hash_attention_topk": topk_tok, "seed": 9}}}
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    rng = rng_for(79)
    NB = B * nblk + 2
    name = "model.layers.1.self_attn.attn"
    k_hash = torch.zeros((NB, BS, 36), dtype=torch.bfloat16, device="cuda")  # 72 bytes per token
    kv_cache = torch.from_numpy(rng.standard_normal((NB, BS, 576)).astype(np.float32)).to(torch.bfloat16).cuda()
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.tensor([nblk * BS, nblk * BS - 100, 9 * BS + 1], dtype=torch.int32, device="cuda")
    # request 0 and 2: prefill through the hook; request 1: first 6 blocks are a prefix-cache hit
    for b in range(B):
        L = int(lens[b])
        first = 6 * BS if b == 1 else 0
        pos = torch.arange(first, L, device="cuda")
        slots = table[b, pos // BS].long() * BS + pos % BS
        lat = kv_cache.view(NB * BS, 576)[slots]
        plugin.set_prefix_cache_hits([(table[b], L, L - first)] if first else [])
        meta = types.SimpleNamespace(slot_mapping=slots)
        layer = types.SimpleNamespace(kv_cache=[kv_cache])
        ctx = types.SimpleNamespace(attn_metadata={name: meta}, no_compile_layers={name: layer}, virtual_engine=0)
        plugin.attention_begin(None, lat[:, :512].contiguous(), lat[:, 512:].contiguous(), name, ctx,
                               phase="prefill", k_hash=k_hash)
    plugin.set_prefix_cache_hits([])
    # every cached token's code = nope code followed by rope code of its latent vector
    codes = k_hash.view(torch.uint8).view(NB * BS, 72)
    flat = kv_cache.view(NB * BS, 576)
    for b in range(B):
        pos = torch.arange(int(lens[b]), device="cuda")
        slots = table[b, pos // BS].long() * BS + pos % BS
        cn, cr = plugin.hash_code(nope=flat[slots, :512].contiguous(), rope=flat[slots, 512:].contiguous())
        assert torch.equal(codes[slots], torch.cat([cn, cr], dim=-1))
    # decode
    ql = torch.from_numpy(rng.standard_normal((B, Hq, 512)).astype(np.float32)).to(torch.bfloat16).cuda()
    qp = torch.from_numpy(rng.standard_normal((B, Hq, 64)).astype(np.float32)).to(torch.bfloat16).cuda()
    pos = lens.long() - 1
    slots = table[torch.arange(B), pos // BS].long() * BS + pos % BS
    lat = flat[slots]
    dec = types.SimpleNamespace(block_table=table.clone(), seq_lens=lens.clone())
    meta = types.SimpleNamespace(slot_mapping=slots, decode=dec)
    ctx = types.SimpleNamespace(attn_metadata={name: meta})
    plugin.attention_begin(None, lat[:, :512].contiguous(), lat[:, 512:].contiguous(), name, ctx,
                           phase="decode", k_hash=k_hash, decode_ql_nope=ql, decode_q_pe=qp)
    kblk = topk_tok // BS
    qn, qr = plugin.hash_code(nope=ql, rope=qp, reduction_head_num=red)
    qc = torch.cat([qn, qr], dim=-1).cpu().numpy().view(np.uint32)          # [B, Hq/red, 18]
    assert qc.shape == (B, Hq // red, 18)
    kc = k_hash.view(torch.uint8).cpu().numpy().view(np.uint32).reshape(NB, BS, 1, 18)
    oi, _ = c_api.hamming_topk(qc, kc, table.cpu().numpy(), lens.cpu().numpy(), kblk, BS, 4 * BS,
                               flags=c_api.F_REDUCE_HEADS | c_api.F_PHYSICAL)
    got = dec.block_table.cpu().numpy()
    assert np.array_equal(got[:, :kblk], np.maximum(oi[:, 0], 0))
    assert not got[:, kblk:].any()
    assert np.array_equal(dec.seq_lens.cpu().numpy(), c_api.update_seq_lens(lens.cpu().numpy(), topk_tok, BS))
    plugin.attention_finished(None, None, None, None, name, ctx, phase="decode")
    assert torch.equal(dec.block_table, table) and torch.equal(dec.seq_lens, lens)


@pytest.mark.parametrize("threshold,red", [(0, 2), (1000, 2), (0, 1), (0, 8)])
def test_plugin_single_call_latent_decode_equals_separate_operators_and_oracle(threshold, red):
    """attention_begin at decode with is_mla as ONE native call (ucm_gsa_decode_step_mla) against the
    same hook running the separate operators (two encode-and-cache calls, two head reductions, two
    hashes, cat, top-k, torch table swap) and against the CPU checker: identical code cache, query
    codes, replacement table and lengths.  Lengths include a request shorter than the top-k budget,
    one shorter than the threshold and a ragged last block."""
    from ucm_amd.sparse.base import UcmSparseFactory, UcmSparseRole

    B, Hq, BS, nblk, topk_tok = 5, 16, 64, 40, 1024
    name = "model.layers.3.self_attn.attn"
    rng = rng_for(93 + red)
    NB = B * nblk + 3
    base_codes = torch.from_numpy(rng.integers(0, 256, size=(NB, BS, 72), dtype=np.uint8)).cuda()
    table = torch.from_numpy(rng.permutation(NB)[: B * nblk].astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.tensor([nblk * BS, nblk * BS - 100, 9 * BS + 1, 700, 17 * BS], dtype=torch.int32, device="cuda")
    ql = torch.from_numpy(rng.standard_normal((B, Hq, 512)).astype(np.float32)).to(torch.bfloat16).cuda()
    qp = torch.from_numpy(rng.standard_normal((B, Hq, 64)).astype(np.float32)).to(torch.bfloat16).cuda()
    lat = torch.from_numpy(rng.standard_normal((B, 576)).astype(np.float32)).to(torch.bfloat16).cuda()
    pos = lens.long() - 1
    slots = table[torch.arange(B), pos // BS].long() * BS + pos % BS
    results = []
    for fused in (True, False):
        cfg = {"ucm_sparse_config": {"GSAOnDevice": {
            "num_q_heads": Hq, "num_kv_heads": 1, "head_dim": 576, "block_size": BS, "is_mla": True,
            "kv_lora_rank": 512, "qk_rope_head_dim": 64, "vllm_hash_attention_reduction_head_num": red,
            "vllm_hash_attention_topk": topk_tok, "gpu_seq_len_threshold": threshold,
            "fused_decode": fused, "seed": 13}}}
        plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
        k_hash = base_codes.clone().view(torch.bfloat16)  # [NB, BS, 36] as the engine allocates it
        dec = types.SimpleNamespace(block_table=table.clone(), seq_lens=lens.clone())
        meta = types.SimpleNamespace(slot_mapping=slots, decode=dec)
        ctx = types.SimpleNamespace(attn_metadata={name: meta})
        for _ in range(2):  # twice: the step's buffers are reused
            plugin.attention_begin(None, lat[:, :512].contiguous(), lat[:, 512:].contiguous(), name, ctx,
                                   phase="decode", k_hash=k_hash, decode_ql_nope=ql, decode_q_pe=qp)
            torch.cuda.synchronize()
            out = (k_hash.clone(), dec.block_table.clone(), dec.seq_lens.clone())
            plugin.attention_finished(None, None, None, None, name, ctx, phase="decode")
            assert torch.equal(dec.block_table, table) and torch.equal(dec.seq_lens, lens)
        results.append((plugin, out))
    (pf, (kh_f, bt_f, sl_f)), (ps, (kh_s, bt_s, sl_s)) = results
    assert len(pf._fused_steps) == 1 and not ps._fused_steps
    assert torch.equal(pf.hash_encoder_nope.hash_weights, ps.hash_encoder_nope.hash_weights)
    # (compared as bytes: as bfloat16 some codes are NaN patterns)
    assert torch.equal(kh_f.view(torch.uint8), kh_s.view(torch.uint8)), \
        "code cache differs between the single call and the separate operators"
    assert not torch.equal(kh_f.view(torch.uint8), base_codes)
    assert torch.equal(bt_f, bt_s) and torch.equal(sl_f, sl_s)
    # the query codes of the single call are the codes of torch's strided head mean
    step = next(iter(pf._fused_steps.values()))
    qn, qr = ps.hash_code(nope=ql, rope=qp, reduction_head_num=red)
    qc_sep = torch.cat([qn, qr], dim=-1).view(torch.int32)
    assert tuple(step.q_codes.shape) == (B, Hq // red, 18)
    assert torch.equal(step.q_codes, qc_sep)
    # and the CPU checker on the codes now in the cache
    kblk = topk_tok // BS
    oi, _ = c_api.hamming_topk(step.q_codes.cpu().numpy().view(np.uint32),
                               kh_f.view(torch.uint8).cpu().numpy().view(np.uint32).reshape(NB, BS, 1, 18),
                               table.cpu().numpy(), lens.cpu().numpy(), kblk, BS, 4 * BS,
                               flags=c_api.F_REDUCE_HEADS | c_api.F_PHYSICAL)
    exp_t = np.zeros((B, nblk), np.int32)
    exp_t[:, :kblk] = np.maximum(oi[:, 0], 0)
    exp_l = c_api.update_seq_lens(lens.cpu().numpy(), topk_tok, BS)
    if threshold:
        short = lens.cpu().numpy() < threshold
        exp_t[short] = table.cpu().numpy()[short]
        exp_l[short] = lens.cpu().numpy()[short]
        assert short.any() and not short.all()
    assert np.array_equal(bt_f.cpu().numpy(), exp_t)
    assert np.array_equal(sl_f.cpu().numpy(), exp_l)


def test_single_call_latent_decode_step_in_a_hip_graph():
    """GSADecodeStepMLA allocates nothing: captured once, replayed with changing inputs and the
    program's own eager work in between, every replay checked against an eager call."""
    from ucm_amd.sparse import GSADecodeStepMLA

    B, Hq, red, BS, nblk, topk_tok = 4, 16, 2, 64, 48, 1024
    rng = rng_for(94)
    NB = B * nblk
    bf = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(torch.bfloat16).cuda()
    wn, wr = bf(512, 512), bf(64, 64)
    cache0 = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(NB, BS, 18), dtype=np.int64).astype(np.int32)).cuda()
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.full((B,), nblk * BS, dtype=torch.int32, device="cuda")
    slots = (table[:, -1].long() * BS + BS - 1)
    ql, qp = torch.empty((B, Hq, 512), dtype=torch.bfloat16, device="cuda"), torch.empty((B, Hq, 64), dtype=torch.bfloat16, device="cuda")
    kn, kr = torch.empty((B, 512), dtype=torch.bfloat16, device="cuda"), torch.empty((B, 64), dtype=torch.bfloat16, device="cuda")
    cache_g, cache_e = cache0.clone(), cache0.clone()
    step = GSADecodeStepMLA(wn, wr, Hq, red, B, nblk, topk_tok, block_size=BS)
    eager = GSADecodeStepMLA(wn, wr, Hq, red, B, nblk, topk_tok, block_size=BS)
    for t in (ql, qp, kn, kr):
        t.copy_(bf(*t.shape))
    step.step(kn, kr, slots, ql, qp, cache_g, table, lens)  # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step.step(kn, kr, slots, ql, qp, cache_g, table, lens)
    for rep in range(4):
        for t in (ql, qp, kn, kr):
            t.copy_(bf(*t.shape))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        et, el = eager.step(kn, kr, slots, ql, qp, cache_e, table, lens)
        torch.cuda.synchronize()
        assert torch.equal(step.new_table, et) and torch.equal(step.new_lens, el), rep
        assert torch.equal(step.q_codes, eager.q_codes) and torch.equal(cache_g, cache_e), rep


def test_host_memory_store_dump_lookup_load_roundtrip():
    """The store contract of the reference's e2e test (ucm/store/test/e2e/cache_on_empty_test.py:
    46-79): dump -> lookup -> load -> bit-exact."""
    from ucm_amd.store import HostMemoryStore

    L, NB, chunk = 4, 16, 8192
    rng = rng_for(88)
    src = [torch.from_numpy(rng.integers(0, 256, size=(2, NB, chunk), dtype=np.uint8)).cuda() for _ in range(L)]
    dst = [torch.zeros_like(t) for t in src]
    store = HostMemoryStore({"tensor_size_list": [chunk] * (2 * L), "capacity_blocks": 8})
    ids = [bytes([i]) * 16 for i in range(5)]
    blocks = [3, 7, 0, 15, 9]
    new_blocks = [1, 2, 4, 5, 6]

    def addrs(tensors, blks):
        return np.array([[t[kv, b].data_ptr() for t in tensors for kv in (0, 1)] for b in blks], np.uint64)

    ev = torch.cuda.Event()
    ev.record()
    task = store.dump_data(ids, [0] * 5, addrs(src, blocks), ev.cuda_event)
    store.wait(task)
    assert store.check(task)
    assert store.lookup(ids + [b"x" * 16]) == [True] * 5 + [False]
    assert store.lookup_on_prefix(ids[:2] + [b"y" * 16] + ids[2:]) == 1
    want = np.concatenate([src[l][kv, blocks[0]].cpu().numpy() for l in range(L) for kv in (0, 1)])
    assert np.array_equal(store.slot_view(ids[0]), want)
    task = store.load_data(ids, [0] * 5, addrs(dst, new_blocks))
    store.wait(task)
    for l in range(L):
        assert torch.equal(dst[l][:, new_blocks], src[l][:, blocks])
        rest = [b for b in range(NB) if b not in new_blocks]
        assert not dst[l][:, rest].any()
    with pytest.raises(RuntimeError):
        store.load_data([b"z" * 16], [0], addrs(dst, [0]))
