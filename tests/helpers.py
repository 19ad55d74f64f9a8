"""Shared test helpers: seeded input builders and the tie-aware comparison rule."""
import numpy as np


def rng_for(seed):
    return np.random.Generator(np.random.PCG64(seed))


def random_codes(rng, shape):
    return rng.integers(0, 2**32, size=shape, dtype=np.uint32)


def make_paged_case(seed, B, Hq, Hkv, Wd, BS, lens, NB=None, extra_blocks=3, table_pad=0,
                    permute=True):
    """Random codes in a paged cache with a seeded permutation block table.
    Returns q [B,Hq,Wd], kc [NB,BS,Hkv,Wd], table [B,max_blocks], lens [B]."""
    rng = rng_for(seed)
    lens = np.asarray(lens, np.int32)
    nblk = [(-(-int(L) // BS)) for L in lens]
    max_blocks = max(max(nblk), 1) + table_pad
    need = int(sum(nblk))
    if NB is None:
        NB = need + extra_blocks
    kc = random_codes(rng, (NB, BS, Hkv, Wd))
    q = random_codes(rng, (B, Hq, Wd))
    phys = rng.permutation(NB) if permute else np.arange(NB)
    table = np.zeros((B, max_blocks), np.int32)
    o = 0
    for b in range(B):
        table[b, : nblk[b]] = phys[o:o + nblk[b]]
        # entries past nblk are junk that must never be dereferenced
        table[b, nblk[b]:] = rng.integers(0, NB, size=max_blocks - nblk[b])
        o += nblk[b]
    return q, kc, table, lens


def assert_topk_matches_unordered_ties(idx, score, ref_idx, ref_score, all_scores=None):
    """The rule for comparing against an implementation whose tie order is unspecified:
    the score sequences must be identical; the index sets must agree for every score value
    strictly better than the last selected one; entries at the boundary score only need to
    be blocks that really have that score (checked when all_scores is given)."""
    idx, score = np.asarray(idx), np.asarray(score)
    ref_idx, ref_score = np.asarray(ref_idx), np.asarray(ref_score)
    assert np.array_equal(np.sort(score), np.sort(ref_score)), (score, ref_score)
    if len(score) == 0:
        return
    boundary = ref_score.max() if all_scores is None else None
    # "worst selected" is the max for distances, which is what the callers pass
    worst = ref_score.max()
    inner = ref_score != worst
    assert set(idx[score != worst].tolist()) == set(ref_idx[inner].tolist())
    if all_scores is not None:
        for i, s in zip(idx.tolist(), score.tolist()):
            assert all_scores[i] == s
    del boundary


def half_piece_sums(q, kc, table, lens, msl):
    """The reference's per-token accumulation (paged_ham_dist_mla.cu:235-241) for one KV head and
    an even code width: per 64-bit piece the integer group-summed popcount is converted to half
    and added in half precision, piece 0 first."""
    B = q.shape[0]
    BS = kc.shape[1]
    kp = np.ascontiguousarray(kc).view(np.uint64)  # [NB,BS,1,L]
    qp = np.ascontiguousarray(q).view(np.uint64)   # [B,G,L]
    cnt = np.array([bin(i).count("1") for i in range(256)], np.int64)
    out = np.full((B, 1, msl), np.inf, np.float16)
    for b in range(B):
        for p in range(min(int(lens[b]), msl)):
            pb = table[b, p // BS]
            if pb < 0 or pb >= kp.shape[0]:
                continue  # unusable entry: infinity
            x = kp[pb, p % BS, 0][None, :] ^ qp[b]          # [G,L]
            parts = cnt[x.view(np.uint8).reshape(x.shape[0], x.shape[1], 8)].sum(axis=(0, 2))
            acc = np.float16(0)
            # sums above 65,504 (128 query heads x 576 bits) overflow to infinity in half
            # precision: that is the reference's own result, not an accident of this helper
            with np.errstate(over="ignore"):
                for part in parts:
                    acc = np.float16(acc + np.float16(part))
            out[b, 0, p] = acc
    return out
