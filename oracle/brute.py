"""Independent numpy / pure-Python restatements for tiny inputs — TEST INFRASTRUCTURE ONLY.

These deliberately use different formulations from ucm_oracle.c so that an index, sign or
transposition mistake in one does not hide in the other:
  * scores come from unpacked +-1 bit vectors and a dot product, the way the reference's own
    self-check does it (csrc/cuda/hash_retrieval/hash_retrieval_worker.py:100-118), through
    sim = (bits + <q_pm, k_pm>) / 2 per query head;
  * top-k is a stable Python sort on (-score, index);
  * the encoder is a float64 matmul followed by numpy.packbits(bitorder="little")
    (hash_encoder.py:359-370 packs with weights 2**arange(8), i.e. LSB first).
"""
import numpy as np


def unpack_pm(codes_u32):
    """uint32 [..., Wd] -> int32 [..., 32*Wd] of +-1; bit n = bit n%32 of word n//32."""
    b = np.ascontiguousarray(codes_u32, dtype="<u4").view(np.uint8)
    bits = np.unpackbits(b, axis=-1, bitorder="little").astype(np.int32)
    return bits * 2 - 1


def hash_encode(x, W):
    """x [M,K], W [K,N] any float -> uint32 [M, N/32], float64 accumulate."""
    p = np.asarray(x, np.float64) @ np.asarray(W, np.float64)
    bits = (p > 0).astype(np.uint8)
    by = np.packbits(bits, axis=-1, bitorder="little")
    return np.ascontiguousarray(by).view("<u4")


def margins(x, W):
    x = np.asarray(x, np.float64)
    p = x @ np.asarray(W, np.float64)
    n = np.linalg.norm(x, axis=-1, keepdims=True)
    return np.abs(p) / np.where(n > 0, n, 1.0)


def block_scores(q, kc, table, lens, sink=0, recent=0):
    """q u32 [B,Hq,Wd]; kc u32 [NB,BS,Hkv,Wd]; table [B,MaxBlk] (required); lens [B].
    -> list over b of int arrays [Hkv, nblk] (similarity form, forced blocks = G*bits)."""
    assert table is not None, "pass an explicit block table (arange for a contiguous cache)"
    B, Hq, Wd = q.shape
    NB, BS, Hkv, _ = kc.shape
    G = Hq // Hkv
    bits = 32 * Wd
    qpm = unpack_pm(q)  # [B,Hq,bits]
    out = []
    for b in range(B):
        L = int(lens[b])
        nblk = -(-L // BS) if L > 0 else 0
        nblk = min(nblk, table.shape[1])
        s = np.zeros((Hkv, nblk), np.int64)
        for j in range(nblk):
            pb = int(table[b, j])
            pos = np.arange(j * BS, min((j + 1) * BS, L))
            forced = bool(np.any(pos < sink) or np.any(pos >= L - recent))
            for h in range(Hkv):
                if pb < 0 or pb >= NB:
                    s[h, j] = -1
                    continue
                if forced:
                    s[h, j] = G * bits
                    continue
                kpm = unpack_pm(kc[pb, : len(pos), h])  # [t,bits]
                qg = qpm[b, h * G:(h + 1) * G]  # [G,bits]
                dots = kpm @ qg.T  # [t,G]
                sim = ((bits + dots) // 2).sum(axis=1)  # exact: bits+dot is even
                s[h, j] = sim.max()
        out.append(s)
    return out


def select_topk(scores_1d, k, score_order=False):
    """Deterministic selection: largest score first, ties to the lower index."""
    n = len(scores_1d)
    order = sorted(range(n), key=lambda j: (-int(scores_1d[j]), j))
    sel = order[: min(k, n)]
    if not score_order:
        sel = sorted(sel)
    return sel


def hamming_topk(q, kc, table, lens, k, sink=0, recent=0, reduce_heads=False, physical=False,
                 score_order=False, distance=False):
    B, Hq, Wd = q.shape
    Hkv = kc.shape[2]
    G = Hq // Hkv
    full = G * 32 * Wd
    Ho = 1 if reduce_heads else Hkv
    idx = -np.ones((B, Ho, k), np.int32)
    sc = np.zeros((B, Ho, k), np.int32)
    bs = block_scores(q, kc, table, lens, sink, recent)
    for b in range(B):
        s = bs[b]
        if s.shape[1] == 0:
            continue
        rows = [s.max(axis=0)] if reduce_heads else [s[h] for h in range(Hkv)]
        for ho, row in enumerate(rows):
            sel = select_topk(row, k, score_order)
            for i, j in enumerate(sel):
                idx[b, ho, i] = int(table[b, j]) if (physical and table is not None) else j
                sc[b, ho, i] = (full - row[j]) if distance else row[j]
    return idx, sc


def update_seq_lens(lens, topk_tok, BS):
    lens = np.asarray(lens, np.int64)
    drop = (np.clip(lens - topk_tok, 0, None) + BS - 1) // BS
    return (lens - drop * BS).astype(np.int32)


def kvstar_block_scores(query_f16, blk_repre_f16, pruned_index=None):
    """float64 restatement of the KVStar block score (simd_compute_kernel.cpp:816-952) with
    library routines: einsum for q.k, a max-shifted softmax over all representatives, a reshape
    and sum per block.  Returns [n_blocks] float64."""
    q = np.asarray(query_f16, np.float16).astype(np.float64)      # [X, Hq, d_orig]
    k = np.asarray(blk_repre_f16, np.float16).astype(np.float64)  # [n, M, Hkv, d]
    n, M, Hkv, d = k.shape
    X, Hq, _ = q.shape
    g = Hq // Hkv
    if pruned_index is not None:
        pr = np.asarray(pruned_index, np.int64)                   # [Hkv, d]
        q = np.stack([q[:, H, pr[H // g]] for H in range(Hq)], axis=1)
    kh = np.repeat(k.reshape(n * M, Hkv, d), g, axis=1)           # [S, Hq, d]
    sc = np.einsum("xhd,shd->xhs", q, kh)
    sc = np.exp(sc - sc.max(axis=2, keepdims=True))
    sc = sc / sc.sum(axis=2, keepdims=True)
    return sc.reshape(X * Hq, n, M).sum(axis=(0, 2))
