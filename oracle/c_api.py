"""ctypes bindings of libucm_oracle.so (the C restatement in ucm_oracle.c).

Test infrastructure only.  All arrays are numpy, contiguous; outputs are new arrays.
"""
import ctypes as C
import importlib.util
import os
import subprocess
import sysconfig

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

F_REDUCE_HEADS, F_PHYSICAL, F_SCORE_ORDER, F_DISTANCE = 1, 2, 4, 8
INF = np.iinfo(np.int32).max


def build(force=False):
    """Compile libucm_oracle.so (and oracle/_ref when the reference checkout exists)."""
    so = os.path.join(_HERE, "libucm_oracle.so")
    if force or not os.path.exists(so):
        subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libucm_oracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
    return _LIB


def ref_backend(name="hash_retrieval_backend"):
    """A CPU retrieval backend of the reference compiled from its own source into oracle/_ref
    (see the Makefile), or None when no build is there.  Names: "hash_retrieval_backend"
    (ucm/sparse/gsa_on_device/csrc/cuda/hash_retrieval/cpy/hash_retrieval_backend.cpp) and
    "retrieval_backend" (ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp)."""
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    path = os.path.join(_HERE, "_ref", name + ext)
    if not os.path.exists(path):
        return None
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def hash_encode(x, W, acc_f64=False, want_margin=False):
    """x [M,K] float32, W [K,N] float32 -> codes uint32 [M,N/32] (+ margin float32 [M,N])."""
    x = _c(x, np.float32)
    W = _c(W, np.float32)
    M, K = x.shape
    N = W.shape[1]
    assert W.shape[0] == K and N % 32 == 0
    codes = np.zeros((M, N // 32), np.uint32)
    margin = np.zeros((M, N), np.float32) if want_margin else None
    lib().oracle_hash_encode(_p(x), C.c_int64(M), C.c_int32(K), _p(W), C.c_int32(N),
                             C.c_int(int(acc_f64)), _p(codes), _p(margin))
    return (codes, margin) if want_margin else codes


def hash_encode_cache(x, W, heads_per_w, slot, cache, BS):
    """x [T,H,K] f32, W [n_w,K,N] f32, slot [T] int, cache uint32 [NB,BS,H,Wd] (modified)."""
    x = _c(x, np.float32)
    W = _c(W, np.float32)
    slot = _c(slot, np.int64)
    assert cache.dtype == np.uint32 and cache.flags.c_contiguous
    T, H, K = x.shape
    n_w, _, N = W.shape
    NB = cache.shape[0]
    st = [s // 4 for s in cache.strides]
    lib().oracle_hash_encode_cache(_p(x), C.c_int64(T), C.c_int32(H), C.c_int32(K), _p(W),
                                   C.c_int32(n_w), C.c_int32(heads_per_w), C.c_int32(N),
                                   _p(slot), _p(cache), C.c_int64(NB), C.c_int32(BS),
                                   C.c_int64(st[0]), C.c_int64(st[1]), C.c_int64(st[2]))
    return cache


def hash_encode_paged(k_cache, block_ids, n_tokens, W, heads_per_w, cache):
    """k_cache [NBk,BS,H,K] f32, block_ids [n] int32, W [n_w,K,N] f32, cache uint32
    [NB,BS,H,Wd] (modified)."""
    k_cache = _c(k_cache, np.float32)
    W = _c(W, np.float32)
    block_ids = _c(block_ids, np.int32)
    assert cache.dtype == np.uint32 and cache.flags.c_contiguous
    NBk, BS, H, K = k_cache.shape
    n_w, _, N = W.shape
    st = [s // 4 for s in cache.strides]
    lib().oracle_hash_encode_paged(_p(k_cache), C.c_int64(NBk), C.c_int32(BS), C.c_int32(H),
                                   C.c_int32(K), _p(block_ids), C.c_int64(n_tokens), _p(W),
                                   C.c_int32(n_w), C.c_int32(heads_per_w), C.c_int32(N), _p(cache),
                                   C.c_int64(cache.shape[0]), C.c_int64(st[0]), C.c_int64(st[1]),
                                   C.c_int64(st[2]))
    return cache


def code_scatter(codes, slot, cache, BS):
    codes = _c(codes, np.uint32)
    slot = _c(slot, np.int64)
    T, H, Wd = codes.shape
    st = [s // 4 for s in cache.strides]
    lib().oracle_code_scatter(_p(codes), C.c_int64(T), C.c_int32(H), C.c_int32(Wd), _p(slot),
                              _p(cache), C.c_int64(cache.shape[0]), C.c_int32(BS),
                              C.c_int64(st[0]), C.c_int64(st[1]), C.c_int64(st[2]))
    return cache


def _cache_args(kc, head_major):
    """kc uint32 [NB,BS,Hkv,Wd] (token-major) or [NB,Hkv,BS,Wd] (head_major)."""
    assert kc.dtype == np.uint32 and kc.flags.c_contiguous
    st = [s // 4 for s in kc.strides]
    if head_major:
        NB, Hkv, BS, Wd = kc.shape
        ks = (st[0], st[2], st[1])
    else:
        NB, BS, Hkv, Wd = kc.shape
        ks = (st[0], st[1], st[2])
    return NB, BS, Hkv, Wd, ks


def hamming_score(q, kc, table, lens, max_seq_len, sink=0, recent=0, reduce_heads=False,
                  head_major=False):
    """Per-token distances int32 [B, Hkv|1, max_seq_len]; INF = int32 max."""
    q = _c(q, np.uint32)
    lens = _c(lens, np.int32)
    NB, BS, Hkv, Wd, ks = _cache_args(kc, head_major)
    B, Hq, _ = q.shape
    if table is not None:
        table = _c(table, np.int32)
        ts, mb = table.shape[1], table.shape[1]
    else:
        ts, mb = 0, (max_seq_len + BS - 1) // BS
    out = np.zeros((B, 1 if reduce_heads else Hkv, max_seq_len), np.int32)
    lib().oracle_hamming_score(_p(q), C.c_int64(Hq * Wd), C.c_int64(Wd), _p(kc), C.c_int64(NB),
                               C.c_int32(BS), C.c_int32(Hkv), C.c_int32(Wd), C.c_int64(ks[0]),
                               C.c_int64(ks[1]), C.c_int64(ks[2]), _p(table), C.c_int32(ts),
                               C.c_int32(mb), _p(lens), C.c_int32(B), C.c_int32(Hq),
                               C.c_int32(max_seq_len), C.c_int32(sink), C.c_int32(recent),
                               C.c_int(int(reduce_heads)), _p(out))
    return out


def hamming_topk(q, kc, table, lens, k, sink=0, recent=0, flags=0, head_major=False,
                 max_blocks=None, nthreads=1, head_items=False):
    """-> (idx, score) int32 [B, Hkv|1, k].  head_items: the threads take (request, KV head)
    items from a shared counter, each pinned to a core (per-head output only)."""
    q = _c(q, np.uint32)
    lens = _c(lens, np.int32)
    NB, BS, Hkv, Wd, ks = _cache_args(kc, head_major)
    B, Hq, _ = q.shape
    if table is not None:
        table = _c(table, np.int32)
        ts = table.shape[1]
        mb = ts if max_blocks is None else max_blocks
    else:
        ts, mb = 0, max_blocks
        assert mb is not None
    Ho = 1 if (flags & F_REDUCE_HEADS) else Hkv
    idx = np.zeros((B, Ho, k), np.int32)
    sc = np.zeros((B, Ho, k), np.int32)
    assert not (head_items and (flags & F_REDUCE_HEADS))
    fn = lib().oracle_hamming_topk_items if head_items else lib().oracle_hamming_topk
    fn(_p(q), C.c_int64(Hq * Wd), C.c_int64(Wd), _p(kc), C.c_int64(NB),
                              C.c_int32(BS), C.c_int32(Hkv), C.c_int32(Wd), C.c_int64(ks[0]),
                              C.c_int64(ks[1]), C.c_int64(ks[2]), _p(table), C.c_int32(ts),
                              C.c_int32(mb), _p(lens), C.c_int32(B), C.c_int32(Hq), C.c_int32(k),
                              C.c_int32(sink), C.c_int32(recent), C.c_uint32(flags), _p(idx),
                              _p(sc), C.c_int32(nthreads))
    return idx, sc


def hash_retrieval(data, query, indexes, k):
    """The reference CPU backend's form: data u8 [NB,BS,dim], query u8 [B,dim],
    indexes i32 [B,max] (-1 = unused).  -> (idx, score, n) with idx/score int32 [B,k]."""
    data = _c(data, np.uint8)
    query = _c(query, np.uint8)
    indexes = _c(indexes, np.int32)
    NB, BS, dim = data.shape
    B = query.shape[0]
    idx = np.zeros((B, k), np.int32)
    sc = np.zeros((B, k), np.int32)
    n = np.zeros((B,), np.int32)
    lib().oracle_hash_retrieval(_p(data), C.c_int64(NB), C.c_int32(BS), C.c_int32(dim),
                                _p(query), C.c_int32(B), _p(indexes),
                                C.c_int32(indexes.shape[1]), C.c_int32(k), _p(idx), _p(sc), _p(n))
    return idx, sc, n


def update_seq_lens(lens, topk_tok, BS):
    lens = _c(lens, np.int32)
    out = np.zeros_like(lens)
    lib().oracle_update_seq_lens(_p(lens), C.c_int32(lens.shape[0]), C.c_int32(topk_tok),
                                 C.c_int32(BS), _p(out))
    return out


def _ptr_array(arrs):
    return np.array([a.ctypes.data for a in arrs], dtype=np.uint64)


def gather(chunks, size):
    """chunks: list of uint8 arrays (>= size bytes each) -> flat uint8 [n*size]."""
    ptrs = _ptr_array(chunks)
    dst = np.zeros(len(chunks) * size, np.uint8)
    lib().oracle_gather(_p(ptrs), _p(dst), C.c_size_t(size), C.c_size_t(len(chunks)))
    return dst


def scatter(flat, chunks, size):
    flat = _c(flat, np.uint8)
    ptrs = _ptr_array(chunks)
    lib().oracle_scatter(_p(flat), _p(ptrs), C.c_size_t(size), C.c_size_t(len(chunks)))


def batch(src_chunks, dst_chunks, size):
    lib().oracle_batch(_p(_ptr_array(src_chunks)), _p(_ptr_array(dst_chunks)), C.c_size_t(size),
                       C.c_size_t(len(src_chunks)))


def block_addrs(base, col_bytes, block_ids):
    base = _c(base, np.uint64)
    col_bytes = _c(col_bytes, np.uint64)
    block_ids = _c(block_ids, np.int32)
    out = np.zeros((block_ids.shape[0], base.shape[0]), np.uint64)
    lib().oracle_block_addrs(_p(base), _p(col_bytes), C.c_int32(base.shape[0]), _p(block_ids),
                             C.c_int64(block_ids.shape[0]), _p(out))
    return out


def paged_copy(base, col_bytes, block_ids, flat, to_cache):
    base = _c(base, np.uint64)
    col_bytes = _c(col_bytes, np.uint64)
    block_ids = _c(block_ids, np.int32)
    assert flat.dtype == np.uint8 and flat.flags.c_contiguous
    lib().oracle_paged_copy(_p(base), _p(col_bytes), C.c_int32(base.shape[0]), _p(block_ids),
                            C.c_int64(block_ids.shape[0]), _p(flat), C.c_int(int(to_cache)))
    return flat


def dot_topk(data, query, indexes, topk):
    """data [n,dim] f32, query [B,dim] f32, indexes [B,max_n] int32 (-1 = none) ->
    (indices int32 [B,topk], scores f32 [B,topk])."""
    data = _c(data, np.float32)
    query = _c(query, np.float32)
    indexes = _c(indexes, np.int32)
    n, dim = data.shape
    B, max_n = indexes.shape
    assert query.shape == (B, dim)
    oi = np.zeros((B, topk), np.int32)
    osc = np.zeros((B, topk), np.float32)
    lib().oracle_dot_topk(_p(data), C.c_int64(n), C.c_int32(dim), _p(query), _p(indexes),
                          C.c_int32(B), C.c_int32(max_n), C.c_int32(topk), _p(oi), _p(osc))
    return oi, osc


def kvstar_topk(query_f16, blk_repre_f16, topk, pruned_index=None):
    """query fp16 [X,Hq,d_orig], blk_repre fp16 [n,M,Hkv,d], pruned_index int64 [Hkv,d] or None
    -> (indices int64 [count], scores f32 [count], all block scores f32 [n])."""
    q = _c(query_f16, np.float16)
    k = _c(blk_repre_f16, np.float16)
    X, Hq, d_orig = q.shape
    n, M, Hkv, d = k.shape
    pr = _c(pruned_index, np.int64) if pruned_index is not None else None
    oi = np.zeros(max(topk, 1), np.int64)
    osc = np.zeros(max(topk, 1), np.float32)
    cnt = C.c_int32(0)
    allsc = np.zeros(n, np.float32)
    lib().oracle_kvstar_topk(_p(q), C.c_int32(X), C.c_int32(Hq), C.c_int32(d_orig), _p(k),
                             C.c_int64(n), C.c_int32(M), C.c_int32(Hkv), C.c_int32(d), _p(pr),
                             C.c_int32(topk), _p(oi), _p(osc), C.byref(cnt), _p(allsc))
    return oi[:cnt.value], osc[:cnt.value], allsc


def half_to_float(bits_u16):
    h = _c(bits_u16, np.uint16)
    out = np.zeros(h.shape, np.float32)
    lib().oracle_half_to_float(_p(h), C.c_int64(h.size), _p(out))
    return out
