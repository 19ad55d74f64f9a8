"""One GQA decode step of the retrieval path in a single native call.

Host-side counterpart of what GSAOnDevice.attention_begin does per layer at decode
(ucm/sparse/gsa_on_device/gsa_on_device.py:850-957): cache_k_hash_gqa_cuda (:564-572) followed
by update_decode_topk_gqa_cuda (:773-786).  All buffers are allocated once in the constructor;
`step` allocates nothing, so it can be captured in a HIP graph.
"""
import torch

from .. import _lib
from .hash_encoder import _DT


class SparseDecodeStep:
    def __init__(self, weights, num_q_heads, num_kv_heads, batch, max_blocks, topk_blocks,
                 block_size=128, sink_token=0, recent_token=0, reduce_heads=False,
                 return_physical=False):
        """weights: [K, N] (shared) or [Hkv, K, N] projection, bf16 / fp16 / fp32, on the GPU."""
        w = weights if weights.dim() == 3 else weights.unsqueeze(0)
        if w.shape[0] not in (1, num_kv_heads):
            raise ValueError("weights must be [K,N] or [Hkv,K,N]")
        if w.dtype not in _DT:
            raise ValueError(f"unsupported weight dtype {w.dtype}")
        self.w = w.contiguous()
        self.K, self.N = int(w.shape[1]), int(w.shape[2])
        if self.N % 32:
            raise ValueError("hash_bits must be a multiple of 32")
        self.Hq, self.Hkv, self.B = int(num_q_heads), int(num_kv_heads), int(batch)
        self.max_blocks, self.k, self.BS = int(max_blocks), int(topk_blocks), int(block_size)
        self.sink, self.recent = int(sink_token), int(recent_token)
        self.flags = ((_lib.TOPK_REDUCE_HEADS if reduce_heads else 0)
                      | (_lib.TOPK_RETURN_PHYSICAL if return_physical else 0))
        dev = w.device
        Ho = 1 if reduce_heads else self.Hkv
        self.q_codes = torch.empty((self.B, self.Hq, self.N // 32), dtype=torch.int32, device=dev)
        self.out_idx = torch.empty((self.B, Ho, self.k), dtype=torch.int32, device=dev)
        self.out_score = torch.empty_like(self.out_idx)
        nbytes = _lib.lib().ucm_hamming_topk_workspace_bytes(self.B, self.Hkv, self.max_blocks)
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def _arguments(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        """Checks the tensors and returns the C call's arguments (all but the stream)."""
        if queries.dtype != self.w.dtype or (new_keys is not None and new_keys.dtype != self.w.dtype):
            raise ValueError("keys, queries and weights must share one dtype")
        if tuple(queries.shape) != (self.B, self.Hq, self.K):
            raise ValueError(f"queries must be {(self.B, self.Hq, self.K)}, got {tuple(queries.shape)}")
        if k_hash_cache.dtype != torch.int32 or k_hash_cache.dim() != 4:
            raise ValueError("k_hash_cache must be int32 [NB,BS,Hkv,W]")
        NB, BS, Hkv, Wd = k_hash_cache.shape
        if BS != self.BS or Hkv != self.Hkv or Wd != self.N // 32:
            raise ValueError("k_hash_cache shape does not match this step's configuration")
        if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
            raise ValueError("block_table and seq_lens must be int32")
        if block_table.shape[0] != self.B or block_table.shape[1] < self.max_blocks:
            raise ValueError("block_table must be [B, >= max_blocks]")
        if queries.stride(-1) != 1 or k_hash_cache.stride(-1) != 1 or block_table.stride(-1) != 1:
            raise ValueError("innermost dimensions must be contiguous")
        T = 0 if new_keys is None else int(new_keys.shape[0])
        if T:
            if tuple(new_keys.shape[1:]) != (self.Hkv, self.K) or new_keys.stride(-1) != 1:
                raise ValueError(f"new_keys must be [T,{self.Hkv},{self.K}] with contiguous rows")
            if slot_mapping.dtype not in (torch.int32, torch.int64) or slot_mapping.numel() != T:
                raise ValueError("slot_mapping must be int32/int64 [T]")
        s = _lib.stride
        return (
            new_keys.data_ptr() if T else None, T, s(new_keys, 0) if T else 0,
            s(new_keys, 1) if T else 0, slot_mapping.data_ptr() if T else None,
            int(T > 0 and slot_mapping.dtype == torch.int64),
            queries.data_ptr(), s(queries, 0), s(queries, 1), _DT[self.w.dtype], self.K,
            self.w.data_ptr(), _DT[self.w.dtype], self.w.shape[0], self.N,
            k_hash_cache.data_ptr(), NB, BS, Hkv, s(k_hash_cache, 0), s(k_hash_cache, 1),
            s(k_hash_cache, 2), block_table.data_ptr(), max(s(block_table, 0), self.max_blocks),
            self.max_blocks, seq_lens.data_ptr(), self.B, self.Hq, self.k, self.sink, self.recent,
            self.flags, self.q_codes.data_ptr(), self.out_idx.data_ptr(), self.out_score.data_ptr(),
            self.workspace.data_ptr(), self.workspace.numel())

    def step(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        """new_keys [T,Hkv,K] + slot_mapping [T] (T may be 0), queries [B,Hq,K],
        k_hash_cache int32 [NB,BS,Hkv,N/32], block_table int32 [B,max_blocks], seq_lens int32 [B].
        Returns (indices, scores) int32 [B, Hkv or 1, k]: views of buffers reused by every call."""
        args = self._arguments(new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        _lib.check(_lib.lib().ucm_sparse_decode_step(*args, _lib.stream_ptr(queries.device)))
        return self.out_idx, self.out_score

    def bind(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        """Validates once and returns `run()`: each call issues the step on torch's current
        stream with the same tensors (whose contents may change between calls) at a few
        microseconds of host time, for serving loops that would otherwise be bound by the
        argument checks.  The tensors must stay alive as long as `run` is used."""
        args = self._arguments(new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        keep = (new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        fn, dev, stream_ptr, check = _lib.lib().ucm_sparse_decode_step, queries.device, _lib.stream_ptr, _lib.check
        result = (self.out_idx, self.out_score)

        def run(_keep=keep):
            check(fn(*args, stream_ptr(dev)))
            return result

        return run


class SparseDecodeStepMLA:
    """One latent-attention (MLA) decode step of the retrieval path in a single native call:
    cache_k_hash_mla_cuda (gsa_on_device.py:426-455) followed by update_decode_topk_mla_cuda
    (:667-709).  The code of a token is the hash of its latent vector (nope) followed by the hash
    of its rope part; the queries are the already head-reduced q_nope / q_pe.  All buffers are
    allocated in the constructor; `step` allocates nothing."""

    def __init__(self, w_nope, w_rope, num_q_heads, batch, max_blocks, topk_blocks, block_size=64,
                 sink_token=0, recent_token=0, return_physical=False):
        """w_nope [K_nope, N_nope], w_rope [K_rope, N_rope]: the two encoders' projections."""
        if w_nope.dtype != w_rope.dtype or w_nope.dtype not in _DT:
            raise ValueError("both projections must share one supported dtype")
        if w_nope.dim() != 2 or w_rope.dim() != 2:
            raise ValueError("projections must be [K, N]")
        self.wn, self.wr = w_nope.contiguous(), w_rope.contiguous()
        self.Kn, self.Nn = (int(v) for v in w_nope.shape)
        self.Kr, self.Nr = (int(v) for v in w_rope.shape)
        if self.Nn % 32 or self.Nr % 32:
            raise ValueError("hash_bits of both parts must be multiples of 32")
        self.Wd = (self.Nn + self.Nr) // 32
        self.Hq, self.B = int(num_q_heads), int(batch)
        self.max_blocks, self.k, self.BS = int(max_blocks), int(topk_blocks), int(block_size)
        self.sink, self.recent = int(sink_token), int(recent_token)
        self.flags = _lib.TOPK_RETURN_PHYSICAL if return_physical else 0
        dev = w_nope.device
        self.q_codes = torch.empty((self.B, self.Hq, self.Wd), dtype=torch.int32, device=dev)
        self.out_idx = torch.empty((self.B, 1, self.k), dtype=torch.int32, device=dev)
        self.out_score = torch.empty_like(self.out_idx)
        nbytes = _lib.lib().ucm_hamming_topk_workspace_bytes(self.B, 1, self.max_blocks)
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def step(self, new_nope, new_rope, slot_mapping, q_nope, q_rope, k_hash_cache, block_table,
             seq_lens):
        """new_nope [T,K_nope], new_rope [T,K_rope] + slot_mapping [T] (T may be 0);
        q_nope [B,Hq,K_nope], q_rope [B,Hq,K_rope]; k_hash_cache int32 [NB,BS,Wd];
        block_table int32 [B,max_blocks]; seq_lens int32 [B].
        Returns (indices, scores) int32 [B, 1, k]: views of buffers reused by every call."""
        dt = self.wn.dtype
        T = 0 if new_nope is None else int(new_nope.shape[0])
        for t in (q_nope, q_rope) + ((new_nope, new_rope) if T else ()):
            if t.dtype != dt or t.stride(-1) != 1:
                raise ValueError("keys, queries and weights must share one dtype and have contiguous rows")
        if tuple(q_nope.shape) != (self.B, self.Hq, self.Kn) or tuple(q_rope.shape) != (self.B, self.Hq, self.Kr):
            raise ValueError("queries must be [B,Hq,K_nope] and [B,Hq,K_rope]")
        if k_hash_cache.dtype != torch.int32 or k_hash_cache.dim() != 3 or k_hash_cache.shape[1] != self.BS \
                or k_hash_cache.shape[2] != self.Wd or k_hash_cache.stride(-1) != 1:
            raise ValueError(f"k_hash_cache must be int32 [NB,{self.BS},{self.Wd}]")
        if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
            raise ValueError("block_table and seq_lens must be int32")
        if block_table.shape[0] != self.B or block_table.shape[1] < self.max_blocks or block_table.stride(-1) != 1:
            raise ValueError("block_table must be [B, >= max_blocks]")
        if T:
            if tuple(new_nope.shape) != (T, self.Kn) or tuple(new_rope.shape) != (T, self.Kr):
                raise ValueError("new keys must be [T,K_nope] and [T,K_rope]")
            if slot_mapping.dtype not in (torch.int32, torch.int64) or slot_mapping.numel() != T:
                raise ValueError("slot_mapping must be int32/int64 [T]")
        s = _lib.stride
        _lib.check(_lib.lib().ucm_sparse_decode_step_mla(
            new_nope.data_ptr() if T else None, s(new_nope, 0) if T else 0,
            new_rope.data_ptr() if T else None, s(new_rope, 0) if T else 0, T,
            slot_mapping.data_ptr() if T else None, int(T > 0 and slot_mapping.dtype == torch.int64),
            q_nope.data_ptr(), s(q_nope, 0), s(q_nope, 1), q_rope.data_ptr(), s(q_rope, 0), s(q_rope, 1),
            _DT[dt], self.Kn, self.Kr, self.wn.data_ptr(), self.wr.data_ptr(), _DT[dt], self.Nn, self.Nr,
            k_hash_cache.data_ptr(), k_hash_cache.shape[0], self.BS, s(k_hash_cache, 0), s(k_hash_cache, 1),
            block_table.data_ptr(), max(s(block_table, 0), self.max_blocks), self.max_blocks,
            seq_lens.data_ptr(), self.B, self.Hq, self.k, self.sink, self.recent, self.flags,
            self.q_codes.data_ptr(), self.out_idx.data_ptr(), self.out_score.data_ptr(),
            self.workspace.data_ptr(), self.workspace.numel(), _lib.stream_ptr(q_nope.device)))
        return self.out_idx, self.out_score


class GSADecodeStep:
    """The GQA plugin's per-layer decode work in one native call (ucm_gsa_decode_step): codes of
    the step's new keys into the paged cache, hash of every KV head's mean query
    (gsa_on_device.py:396-412), block scores with the best KV head counting and sink / recent
    blocks kept (hamming_topk.py:15-54), and the replacement block table and sequence lengths
    the attention backend reads (gsa_on_device.py:786-811).  Buffers are allocated once here;
    `step` allocates nothing and can be captured in a HIP graph."""

    def __init__(self, weights, num_q_heads, num_kv_heads, batch, table_width, topk_tokens,
                 block_size=128, sink_token=None, recent_token=None, seq_len_threshold=0):
        w = weights if weights.dim() == 3 else weights.unsqueeze(0)
        if w.shape[0] not in (1, num_kv_heads):
            raise ValueError("weights must be [K,N] or [Hkv,K,N]")
        if w.dtype not in _DT or w.dtype == torch.float32:
            raise ValueError("the fused step needs bfloat16 or float16 weights")
        self.w = w.contiguous()
        self.K, self.N = int(w.shape[1]), int(w.shape[2])
        self.Hq, self.Hkv, self.B = int(num_q_heads), int(num_kv_heads), int(batch)
        self.width, self.BS = int(table_width), int(block_size)
        self.topk = int(topk_tokens)
        self.sink = self.BS if sink_token is None else int(sink_token)
        self.recent = 4 * self.BS if recent_token is None else int(recent_token)
        self.threshold = int(seq_len_threshold)
        assert self.topk % self.BS == 0
        assert self.recent > 0 and self.topk > self.sink + self.recent
        dev = w.device
        self.q_codes = torch.empty((self.B, self.Hkv, self.N // 32), dtype=torch.int32, device=dev)
        self.new_table = torch.empty((self.B, self.width), dtype=torch.int32, device=dev)
        self.new_lens = torch.empty((self.B,), dtype=torch.int32, device=dev)
        nbytes = _lib.lib().ucm_hamming_topk_workspace_bytes(self.B, self.Hkv, self.width)
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def _arguments(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        if queries.dtype != self.w.dtype or (new_keys is not None and new_keys.dtype != self.w.dtype):
            raise ValueError("keys, queries and weights must share one dtype")
        if tuple(queries.shape) != (self.B, self.Hq, self.K) or queries.stride(-1) != 1:
            raise ValueError(f"queries must be {(self.B, self.Hq, self.K)} with contiguous rows")
        if k_hash_cache.dtype != torch.int32 or k_hash_cache.dim() != 4 or k_hash_cache.stride(-1) != 1:
            raise ValueError("k_hash_cache must be int32 [NB,BS,Hkv,W]")
        NB, BS, Hkv, Wd = k_hash_cache.shape
        if BS != self.BS or Hkv != self.Hkv or Wd != self.N // 32:
            raise ValueError("k_hash_cache shape does not match this step's configuration")
        if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
            raise ValueError("block_table and seq_lens must be int32")
        if tuple(block_table.shape) != (self.B, self.width) or block_table.stride(-1) != 1:
            raise ValueError(f"block_table must be {(self.B, self.width)}")
        if seq_lens.numel() != self.B or not seq_lens.is_contiguous():
            raise ValueError("seq_lens must be a contiguous [B] tensor")
        T = 0 if new_keys is None else int(new_keys.shape[0])
        if T:
            if tuple(new_keys.shape[1:]) != (self.Hkv, self.K) or new_keys.stride(-1) != 1:
                raise ValueError(f"new_keys must be [T,{self.Hkv},{self.K}] with contiguous rows")
            if slot_mapping.dtype not in (torch.int32, torch.int64) or slot_mapping.numel() != T \
                    or not slot_mapping.is_contiguous():
                raise ValueError("slot_mapping must be a contiguous int32/int64 [T] tensor")
        s = _lib.stride
        return (
            new_keys.data_ptr() if T else None, T, s(new_keys, 0) if T else 0,
            s(new_keys, 1) if T else 0, slot_mapping.data_ptr() if T else None,
            int(T > 0 and slot_mapping.dtype == torch.int64),
            queries.data_ptr(), s(queries, 0), s(queries, 1), _DT[self.w.dtype], self.K,
            self.w.data_ptr(), _DT[self.w.dtype], self.w.shape[0], self.N,
            k_hash_cache.data_ptr(), NB, BS, Hkv, s(k_hash_cache, 0), s(k_hash_cache, 1),
            s(k_hash_cache, 2), block_table.data_ptr(), max(s(block_table, 0), self.width),
            self.width, seq_lens.data_ptr(), self.B, self.Hq, self.topk, self.sink, self.recent,
            self.threshold, self.q_codes.data_ptr(), self.new_table.data_ptr(), self.width,
            self.new_lens.data_ptr(), self.workspace.data_ptr(), self.workspace.numel())

    def step(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        """Returns (new_block_table [B, width], new_seq_lens [B]): buffers reused by every call."""
        args = self._arguments(new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        _lib.check(_lib.lib().ucm_gsa_decode_step(*args, _lib.stream_ptr(queries.device)))
        return self.new_table, self.new_lens

    def bind(self, new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens):
        """Validates once; the returned `run()` reissues the step with the same tensors."""
        args = self._arguments(new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        keep = (new_keys, slot_mapping, queries, k_hash_cache, block_table, seq_lens)
        fn, dev, stream_ptr, check = _lib.lib().ucm_gsa_decode_step, queries.device, _lib.stream_ptr, _lib.check
        result = (self.new_table, self.new_lens)

        def run(_keep=keep):
            check(fn(*args, stream_ptr(dev)))
            return result

        return run


class GSADecodeStepMLA:
    """The latent-attention plugin's per-layer decode work in one native call
    (ucm_gsa_decode_step_mla): both parts of the step's new latent keys into the paged code cache
    (cache_k_hash_mla_cuda, gsa_on_device.py:426-455), the head reduction and both hashes of the
    queries (hash_code, :376-393), block scores with sink / recent blocks kept and the selection
    (update_decode_topk_mla_cuda, :667-709), and the replacement block table and sequence lengths
    the attention backend reads.  Buffers are allocated once here; `step` allocates nothing and
    can be captured in a HIP graph."""

    def __init__(self, w_nope, w_rope, num_q_heads, reduction_head_num, batch, table_width, topk_tokens,
                 block_size=64, sink_token=None, recent_token=None, seq_len_threshold=0):
        if w_nope.dtype != w_rope.dtype or w_nope.dtype not in _DT or w_nope.dtype == torch.float32:
            raise ValueError("the fused step needs two bfloat16 or float16 projections of one dtype")
        if w_nope.dim() != 2 or w_rope.dim() != 2:
            raise ValueError("projections must be [K, N]")
        self.wn, self.wr = w_nope.contiguous(), w_rope.contiguous()
        self.Kn, self.Nn = (int(v) for v in w_nope.shape)
        self.Kr, self.Nr = (int(v) for v in w_rope.shape)
        if self.Nn % 32 or self.Nr % 32:
            raise ValueError("hash_bits of both parts must be multiples of 32")
        self.Wd = (self.Nn + self.Nr) // 32
        self.Hq, self.R, self.B = int(num_q_heads), max(1, int(reduction_head_num)), int(batch)
        if self.Hq % self.R:
            raise ValueError(f"{self.Hq} query heads do not reduce by {self.R}")
        self.width, self.BS, self.topk = int(table_width), int(block_size), int(topk_tokens)
        self.sink = self.BS if sink_token is None else int(sink_token)
        self.recent = 4 * self.BS if recent_token is None else int(recent_token)
        self.threshold = int(seq_len_threshold)
        assert self.topk % self.BS == 0
        assert self.recent > 0 and self.topk > self.sink + self.recent
        dev = w_nope.device
        self.q_codes = torch.empty((self.B, self.Hq // self.R, self.Wd), dtype=torch.int32, device=dev)
        self.new_table = torch.empty((self.B, self.width), dtype=torch.int32, device=dev)
        self.new_lens = torch.empty((self.B,), dtype=torch.int32, device=dev)
        nbytes = _lib.lib().ucm_hamming_topk_workspace_bytes(self.B, 1, self.width)
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def step(self, new_nope, new_rope, slot_mapping, q_nope, q_rope, k_hash_cache, block_table, seq_lens):
        """new_nope [T,K_nope], new_rope [T,K_rope] + slot_mapping [T] (T may be 0); q_nope
        [B,Hq,K_nope], q_rope [B,Hq,K_rope] (all Hq heads: the reduction happens inside);
        k_hash_cache int32 [NB,BS,Wd]; block_table int32 [B,width]; seq_lens int32 [B].
        Returns (new_block_table [B, width], new_seq_lens [B]): buffers reused by every call."""
        dt = self.wn.dtype
        T = 0 if new_nope is None else int(new_nope.shape[0])
        for t in (q_nope, q_rope) + ((new_nope, new_rope) if T else ()):
            if t.dtype != dt or t.stride(-1) != 1:
                raise ValueError("keys, queries and weights must share one dtype and have contiguous rows")
        if tuple(q_nope.shape) != (self.B, self.Hq, self.Kn) or tuple(q_rope.shape) != (self.B, self.Hq, self.Kr):
            raise ValueError("queries must be [B,Hq,K_nope] and [B,Hq,K_rope]")
        if k_hash_cache.dtype != torch.int32 or k_hash_cache.dim() != 3 or k_hash_cache.shape[1] != self.BS \
                or k_hash_cache.shape[2] != self.Wd or k_hash_cache.stride(-1) != 1:
            raise ValueError(f"k_hash_cache must be int32 [NB,{self.BS},{self.Wd}]")
        if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
            raise ValueError("block_table and seq_lens must be int32")
        if tuple(block_table.shape) != (self.B, self.width) or block_table.stride(-1) != 1:
            raise ValueError(f"block_table must be {(self.B, self.width)}")
        if seq_lens.numel() != self.B or not seq_lens.is_contiguous():
            raise ValueError("seq_lens must be a contiguous [B] tensor")
        if T:
            if tuple(new_nope.shape) != (T, self.Kn) or tuple(new_rope.shape) != (T, self.Kr):
                raise ValueError("new keys must be [T,K_nope] and [T,K_rope]")
            if slot_mapping.dtype not in (torch.int32, torch.int64) or slot_mapping.numel() != T \
                    or not slot_mapping.is_contiguous():
                raise ValueError("slot_mapping must be a contiguous int32/int64 [T] tensor")
        s = _lib.stride
        _lib.check(_lib.lib().ucm_gsa_decode_step_mla(
            new_nope.data_ptr() if T else None, s(new_nope, 0) if T else 0,
            new_rope.data_ptr() if T else None, s(new_rope, 0) if T else 0, T,
            slot_mapping.data_ptr() if T else None, int(T > 0 and slot_mapping.dtype == torch.int64),
            q_nope.data_ptr(), s(q_nope, 0), s(q_nope, 1), q_rope.data_ptr(), s(q_rope, 0), s(q_rope, 1),
            _DT[dt], self.Kn, self.Kr, self.wn.data_ptr(), self.wr.data_ptr(), _DT[dt], self.Nn, self.Nr,
            k_hash_cache.data_ptr(), k_hash_cache.shape[0], self.BS, s(k_hash_cache, 0), s(k_hash_cache, 1),
            block_table.data_ptr(), max(s(block_table, 0), self.width), self.width,
            seq_lens.data_ptr(), self.B, self.Hq, self.R, self.topk, self.sink, self.recent, self.threshold,
            self.q_codes.data_ptr(), self.new_table.data_ptr(), self.width, self.new_lens.data_ptr(),
            self.workspace.data_ptr(), self.workspace.numel(), _lib.stream_ptr(q_nope.device)))
        return self.new_table, self.new_lens
