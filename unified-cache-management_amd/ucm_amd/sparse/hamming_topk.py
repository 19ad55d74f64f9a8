"""Hamming block top-k on MI355X behind the reference's call surface.

Mirrors ucm/sparse/gsa_on_device/hamming_topk.py (update_seq_lens, cuda_hamming_topk) and
the `hamming.hamming_score` binding (csrc/cuda/ham_dist/cpy/hamming.cpp:4-6), plus the full
operator `hamming_topk` with per-KV-head int32 scores (the contract of the reference's NPU op,
csrc/ascend/torch_binding.cpp:39-57).
"""
import torch

from .. import _lib

_workspaces = {}
_retired = []


def _workspace(device, nbytes):
    """Scratch of the calling stream.  One buffer per (device, stream): calls on different
    streams (a retrieval worker's side stream beside the plugin on the main stream) may be in
    flight together and must not share block scores.  A buffer that is outgrown stays alive
    (kernels already enqueued, or a captured graph, may still use it); sizes double, so the
    retired ones add up to less than the live one."""
    stream = torch.cuda.current_stream(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(),
           stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        size = max(nbytes, 1 << 20, 2 * ws.numel() if ws is not None else 0)
        ws = torch.empty(size, dtype=torch.uint8, device=device)  # allocated on `stream`
        _workspaces[key] = ws
    return ws


def _as_words(t, name):
    """View a code tensor (uint8 / bf16 / int32 ...) as int32 words over the last dim."""
    if t.dtype == torch.int32:
        return t
    if t.stride(-1) != 1:
        t = t.contiguous()
    if (t.shape[-1] * t.element_size()) % 4:
        raise ValueError(f"{name}: codes must be a whole number of 32-bit words")
    return t.view(torch.int32)


def update_seq_lens(seq_lens, topk_token, block_size):
    """seq_lens - ceil(max(seq_lens - topk_token, 0) / block_size) * block_size
    (hamming_topk.py:7-12), computed on the device by the library."""
    s = seq_lens.contiguous()
    if s.dtype != torch.int32:
        s = s.to(torch.int32)
    out = torch.empty_like(s)
    _lib.check(_lib.lib().ucm_update_seq_lens(s.data_ptr(), s.numel(), int(topk_token),
                                              int(block_size), out.data_ptr(),
                                              _lib.stream_ptr(s.device)))
    return out.to(seq_lens.dtype)


def _cache_geometry(k_hash, head_major):
    st = [_lib.stride(k_hash, d) for d in range(4)]
    if st[3] != 1:
        raise ValueError("key codes must be contiguous in the last dimension")
    if head_major:
        NB, Hkv, BS, Wd = k_hash.shape
        return NB, BS, Hkv, Wd, (st[0], st[2], st[1])
    NB, BS, Hkv, Wd = k_hash.shape
    return NB, BS, Hkv, Wd, (st[0], st[1], st[2])


def _common(q_hash, k_hash, block_table, seq_lens, head_major):
    q = _as_words(q_hash, "q_hash")
    k = _as_words(k_hash, "k_hash")
    if k.ndim != 4:
        raise ValueError(f"k_hash must be rank-4, got {tuple(k.shape)}")
    if q.ndim == 4:  # [B, 1, Hq, W] as the reference passes it
        if q.shape[1] != 1:
            raise ValueError("q_hash [B, Sq, Hq, W] needs Sq == 1")
        q = q[:, 0]
    if q.ndim != 3:
        raise ValueError(f"q_hash must be [B,Hq,W] or [B,1,Hq,W], got {tuple(q.shape)}")
    if q.stride(-1) != 1:
        q = q.contiguous()
    NB, BS, Hkv, Wd, ks = _cache_geometry(k, head_major)
    B, Hq, Wq = q.shape
    if Wq != Wd:
        raise ValueError(f"code width mismatch: query {Wq} words, keys {Wd} words")
    if block_table is not None:
        if block_table.dtype != torch.int32:
            raise ValueError("block_table must be int32")
        if block_table.shape[0] != B:
            raise ValueError("batch size mismatch between query_code and block_table")
        if block_table.stride(-1) != 1:
            block_table = block_table.contiguous()
    if seq_lens.dtype != torch.int32:
        raise ValueError("seq_lens must be int32")
    seq_lens = seq_lens.contiguous()
    if seq_lens.numel() != B:
        raise ValueError("seq_lens must have one entry per request")
    for t in (k, block_table, seq_lens):
        if t is not None and t.device != q.device:
            raise ValueError("all tensors must be on the same device")
    if q.device.type != "cuda":
        raise ValueError("the HIP library needs tensors on a GPU device")
    return q, k, block_table, seq_lens, (NB, BS, Hkv, Wd, ks, B, Hq)


def hamming_topk(q_hash, k_hash, block_table, seq_lens, k_blocks, sink_token=0, recent_token=0, *,
                 reduce_heads=False, return_physical=False, score_order=False, distance=False,
                 head_major=False, max_blocks=None, with_scores=True):
    """Top-k blocks per (request, KV head).

    q_hash      [B,Hq,W] (or [B,1,Hq,W]) packed codes, any element type that views as int32
    k_hash      [NB,BS,Hkv,W] paged codes ([NB,Hkv,BS,W] with head_major=True)
    block_table int32 [B,max_blocks] or None (contiguous cache: request b owns blocks
                b*max_blocks..)
    seq_lens    int32 [B]
    Returns (indices, scores) int32 [B, Hkv or 1, k_blocks]; unused slots -1 / 0.  Score =
    sum over the GQA group of (bits - popcount(q xor k)), max over the block's valid tokens;
    ties go to the lower block index; indices ascend unless score_order=True.
    """
    q, k, block_table, seq_lens, (NB, BS, Hkv, Wd, ks, B, Hq) = _common(
        q_hash, k_hash, block_table, seq_lens, head_major)
    if block_table is not None:
        mb = block_table.shape[1] if max_blocks is None else int(max_blocks)
        ts = max(_lib.stride(block_table, 0), mb)
    else:
        if max_blocks is None:
            raise ValueError("max_blocks is required without a block table")
        mb, ts = int(max_blocks), 0
    flags = ((_lib.TOPK_REDUCE_HEADS if reduce_heads else 0)
             | (_lib.TOPK_RETURN_PHYSICAL if return_physical else 0)
             | (_lib.TOPK_SCORE_ORDER if score_order else 0)
             | (_lib.TOPK_DISTANCE if distance else 0))
    Ho = 1 if reduce_heads else Hkv
    idx = torch.empty((B, Ho, int(k_blocks)), dtype=torch.int32, device=q.device)
    sc = torch.empty_like(idx) if with_scores else None
    L = _lib.lib()
    nbytes = L.ucm_hamming_topk_workspace_bytes(B, Hkv, mb)
    ws = _workspace(q.device, nbytes)
    _lib.check(L.ucm_hamming_topk(
        q.data_ptr(), _lib.stride(q, 0), _lib.stride(q, 1), k.data_ptr(), NB, BS, Hkv, Wd, ks[0], ks[1], ks[2],
        block_table.data_ptr() if block_table is not None else None, ts, mb, seq_lens.data_ptr(),
        B, Hq, int(k_blocks), int(sink_token), int(recent_token), flags, idx.data_ptr(),
        sc.data_ptr() if sc is not None else None, ws.data_ptr(), ws.numel(),
        _lib.stream_ptr(q.device)))
    return idx, sc


def hamming_score(key_codes, query_code, block_table, seq_len, max_seq_len, sink, recent,
                  reduce_kvhead, out_int32=False):
    """Per-token group-summed Hamming distance, the output of the reference's scorer
    (kvlib::HammingScoreContiCUDA, csrc/cuda/ham_dist/paged_ham_dist_mla.cu:332-443):
    float16 [B, Hkv or 1, max_seq_len]; 0 at sink/recent positions, +inf past seq_len.
    out_int32=True returns exact int32 distances (inf = int32 max) instead.

    block_table=None is the reference's contiguous form (paged_ham_dist_mla.cu:345,444-):
    key_codes is [B, S, Hkv, C] and position p of request b is key_codes[b, p].  The codes are
    then read as blocks of the largest power of two up to 128 that divides S, block j of request b
    at b * (S / block) + j, which is the library's table-free addressing."""
    if block_table is None:
        kw = _as_words(key_codes, "key_codes")
        if kw.ndim != 4:
            raise ValueError(f"key_codes must be [B,S,Hkv,C], got {tuple(kw.shape)}")
        kw = kw.contiguous()
        Bk, S, Hk, C = kw.shape
        bsv = 128
        while S % bsv:
            bsv //= 2
        key_codes = kw.view(Bk * (S // bsv), bsv, Hk, C)
        n_table_blocks = S // bsv
    q, k, block_table, seq_len, (NB, BS, Hkv, Wd, ks, B, Hq) = _common(
        query_code, key_codes, block_table, seq_len, False)
    if block_table is None:
        if NB != B * n_table_blocks:
            raise ValueError("batch size mismatch between query_code and key_codes")
        table_ptr, table_stride, max_blocks = None, 0, n_table_blocks
    else:
        table_ptr = block_table.data_ptr()
        table_stride = max(_lib.stride(block_table, 0), block_table.shape[1])
        max_blocks = block_table.shape[1]
    Ho = 1 if reduce_kvhead else Hkv
    out = torch.empty((B, Ho, int(max_seq_len)),
                      dtype=torch.int32 if out_int32 else torch.float16, device=q.device)
    ws = torch.empty(_lib.lib().ucm_hamming_score_workspace_bytes(B, Hq, Wd), dtype=torch.uint8,
                     device=q.device)
    _lib.check(_lib.lib().ucm_hamming_score(
        q.data_ptr(), _lib.stride(q, 0), _lib.stride(q, 1), k.data_ptr(), NB, BS, Hkv, Wd, ks[0], ks[1], ks[2],
        table_ptr, table_stride, max_blocks, seq_len.data_ptr(),
        B, Hq, int(max_seq_len), int(sink), int(recent), int(bool(reduce_kvhead)), out.data_ptr(),
        int(not out_int32), ws.data_ptr(), ws.numel(), _lib.stream_ptr(q.device)))
    return out


def cuda_hamming_topk(q_hash, k_hash, block_table, seq_lens, topk_token, sink_token, recent_token,
                      is_mla):
    """Drop-in for the reference's cuda_hamming_topk (hamming_topk.py:15-54): returns the
    physical ids of the topk_token // block_size best blocks per request, in logical order.
    One list per request: KV heads are min-reduced unless is_mla (hamming_topk.py:33).
    Slots beyond a request's block count hold 0 (the filler the plugin itself uses,
    gsa_on_device.py:790)."""
    k = _as_words(k_hash, "k_hash")
    block_size = k.shape[1]
    assert topk_token % block_size == 0
    assert recent_token > 0 and topk_token > (sink_token + recent_token)
    reduce_kvhead = (not is_mla) and (k.size(2) > 1)
    idx, _ = hamming_topk(q_hash, k, block_table, seq_lens, topk_token // block_size, sink_token,
                          recent_token, reduce_heads=reduce_kvhead or k.size(2) == 1,
                          return_physical=True, with_scores=False)
    return idx[:, 0].clamp_(min=0)
