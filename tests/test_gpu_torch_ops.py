"""GPU: the operators registered with PyTorch's dispatcher (torch.ops.ucm_amd.*) against the CPU
checker and the ctypes mirror - same library, same kernels, bit-exact."""
import numpy as np
import pytest
import torch

from helpers import make_paged_case, rng_for
from oracle import brute, c_api

pytestmark = pytest.mark.gpu


def _dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.cuda()


@pytest.mark.parametrize("flags", [0, 1 | 2])
def test_hamming_topk_operator_matches_the_checker(flags):
    from ucm_amd import torch_ops

    ops = torch_ops.load()
    B, Hq, Hkv, Wd, BS, k = 3, 32, 8, 4, 128, 16
    q, kc, table, lens = make_paged_case(501, B, Hq, Hkv, Wd, BS, [8192, 5000, 129])
    idx, sc = ops.hamming_topk(_dev(q), _dev(kc), _dev(table), _dev(lens), k, 0, 0, flags)
    torch.cuda.synchronize()
    oi, os_ = c_api.hamming_topk(q, kc, table, lens, k, 0, 0, flags)
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.array_equal(sc.cpu().numpy(), os_)


def test_hash_encode_cache_operator_matches_the_mirror_and_the_margin_rule():
    from ucm_amd import torch_ops
    from ucm_amd.sparse import HashEncoder

    ops = torch_ops.load()
    rng = rng_for(502)
    T, H, K, N, BS, NB = 700, 8, 128, 128, 16, 50
    x = torch.from_numpy(rng.standard_normal((T, H, K)).astype(np.float32)).to(torch.bfloat16).cuda()
    w = torch.from_numpy(rng.standard_normal((H, K, N)).astype(np.float32)).to(torch.bfloat16).cuda()
    slots = torch.from_numpy(rng.permutation(NB * BS)[:T].astype(np.int64)).cuda()
    cache = torch.full((NB, BS, H, N // 32), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    ops.hash_encode_cache(x, w, slots, cache)
    enc = HashEncoder(K, N, torch.bfloat16, torch.device("cuda"), num_weights=H, heads_per_weight=1)
    enc.set_hash_weight(w)
    ref = torch.full_like(cache, 0x5A5A5A5A)
    enc.compute_hash_and_cache(x, slots, ref, block_size=BS)
    torch.cuda.synchronize()
    assert torch.equal(cache, ref)
    got = cache.cpu().numpy().view(np.uint32).reshape(NB * BS, H, N // 32)[slots.cpu().numpy()]
    xs, ws = x.float().cpu().numpy(), w.float().cpu().numpy()
    for h in range(H):
        exp = brute.hash_encode(xs[:, h], ws[h])
        diff = np.unpackbits((got[:, h] ^ exp).view(np.uint8), axis=-1, bitorder="little").astype(bool)
        assert not np.any(diff & (brute.margins(xs[:, h], ws[h]) >= 1e-2))


def test_gsa_decode_step_operator_matches_the_mirror():
    from ucm_amd import torch_ops
    from ucm_amd.sparse import GSADecodeStep

    ops = torch_ops.load()
    rng = rng_for(503)
    B, Hq, Hkv, D, BS, nblk, topk_tok = 4, 32, 8, 128, 128, 24, 1024
    NB = B * nblk
    w = torch.from_numpy(rng.standard_normal((D, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    cache = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, size=(NB, BS, Hkv, D // 32), dtype=np.int64)
                             .astype(np.int32)).cuda()
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32).reshape(B, nblk)).cuda()
    lens = torch.tensor([nblk * BS, nblk * BS - 77, 1500, 9 * BS + 1], dtype=torch.int32, device="cuda")
    q = torch.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    newk = torch.from_numpy(rng.standard_normal((B, Hkv, D)).astype(np.float32)).to(torch.bfloat16).cuda()
    pos = lens.long() - 1
    slots = table[torch.arange(B), pos // BS].long() * BS + pos % BS
    c_op, c_ref = cache.clone(), cache.clone()
    nt, nl = ops.gsa_decode_step(newk, slots, q, w, c_op, table, lens, topk_tok, BS, 4 * BS, 2000)
    step = GSADecodeStep(w, Hq, Hkv, B, nblk, topk_tok, block_size=BS, seq_len_threshold=2000)
    rt, rl = step.step(newk, slots, q, c_ref, table, lens)
    torch.cuda.synchronize()
    assert torch.equal(c_op, c_ref) and not torch.equal(c_op, cache)
    assert torch.equal(nt, rt) and torch.equal(nl, rl)
