"""GSAOnDevice-shaped driver of the MI355X operators (GQA and latent-attention decode paths).

A thin counterpart of the reference plugin's worker-side hot path
(ucm/sparse/gsa_on_device/gsa_on_device.py): `attention_begin` stores the hash codes of the
step's keys (cache_k_hash_gqa_cuda, :564-572) and, at decode, replaces the layer's block table
and seq_lens with the top-k blocks (update_decode_topk_gqa_cuda, :773-811);
`attention_finished` puts the originals back (:959-995).  Engine metadata is duck-typed: the
layer's `attn_metadata` needs `slot_mapping`, `block_table` and `seq_lens` attributes.
After a prefix-cache hit (`set_prefix_cache_hits`, the bookkeeping of build_sparse_meta,
:1322-1366) the keys that were loaded into the paged KV cache are re-encoded in place
(cache_k_hash_gqa_cuda's `has_pc_hit` branch, :574-588).  With `is_mla` the keys are the latent
vector (nope, kv_lora_rank values) and the rope part (qk_rope_head_dim values) of one KV head:
two encoders write their codes side by side into 18-word cache rows (cache_k_hash_mla_cuda,
:426-455 — the fused encode-and-store takes the place of hash + vLLM's concat_and_cache_mla),
and the decode query codes of the, optionally head-reduced, q_nope / q_pe are compared against
them (update_decode_topk_mla_cuda, :667-709).  The scheduler-side hooks, the FlashMLA tile
metadata swap and layer-skip profiling of the reference are outside this build.

Configuration (`ucm_sparse_config["GSAOnDevice"]`), names from
gsa_on_device_config.py:36-98 where they exist:
    num_q_heads, num_kv_heads, head_dim, block_size, hash_bits (default head_dim),
    vllm_hash_attention_topk (tokens kept), sink_tokens (default block_size),
    recent_tokens (default 4 * block_size), vllm_hash_attention_rollback_layers,
    gpu_seq_len_threshold, dtype ("bfloat16"|"float16"|"float32"), device, seed;
    is_mla, kv_lora_rank (512), qk_rope_head_dim (64), vllm_hash_attention_reduction_head_num
"""
from typing import List, Optional, Union

import torch

from .base import UcmSparseBase, UcmSparseMetadata, UcmSparseRole
from .decode_step import GSADecodeStep, GSADecodeStepMLA
from .hamming_topk import _as_words, cuda_hamming_topk, update_seq_lens
from .hash_encoder import HashEncoder

_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


class GSAOnDeviceMetadata(UcmSparseMetadata):
    pass


class GSAOnDevice(UcmSparseBase):
    def __init__(self, vllm_config, role: UcmSparseRole):
        super().__init__(vllm_config, role)
        cfg = getattr(vllm_config, "ucm_sparse_config", None)
        if cfg is None:
            cfg = vllm_config["ucm_sparse_config"]
        cfg = cfg["GSAOnDevice"]
        self.num_q_heads = int(cfg["num_q_heads"])
        self.num_key_heads = int(cfg["num_kv_heads"])
        self.head_dim = int(cfg["head_dim"])
        self.block_size = int(cfg.get("block_size", 128))
        self.hash_bits = int(cfg.get("hash_bits", self.head_dim))
        self.hash_topk_tokens = int(cfg.get("vllm_hash_attention_topk", 2048))
        self.sink_tokens = int(cfg.get("sink_tokens", self.block_size))
        self.recent_tokens = int(cfg.get("recent_tokens", 4 * self.block_size))
        self.hash_rollback_layers = list(cfg.get("vllm_hash_attention_rollback_layers", []))
        self.seq_len_threshold = int(cfg.get("gpu_seq_len_threshold", 0))
        self.device = torch.device(cfg.get("device", "cuda:0"))
        self.dtype = _DTYPES[cfg.get("dtype", "bfloat16")]
        if "seed" in cfg:
            torch.manual_seed(int(cfg["seed"]))
        self.is_mla = bool(cfg.get("is_mla", False))
        self.gsa_enabled = True
        if self.is_mla:
            # gsa_on_device.py:210-232: one encoder per part, as many bits as dimensions
            self.hash_reduction_head_num = cfg.get("vllm_hash_attention_reduction_head_num") or 1
            self.kv_lora_rank = int(cfg.get("kv_lora_rank", 512))
            self.qk_rope_head_dim = int(cfg.get("qk_rope_head_dim", 64))
            self.hash_encoder_nope = HashEncoder(self.kv_lora_rank, self.kv_lora_rank, self.dtype,
                                                 self.device)
            self.hash_encoder_rope = HashEncoder(self.qk_rope_head_dim, self.qk_rope_head_dim,
                                                 self.dtype, self.device)
            self.hash_encoder = None
        else:
            self.hash_encoder = HashEncoder(self.head_dim, self.hash_bits, self.dtype, self.device)
        self._saved = {}
        self._fused_steps = {}  # (requests, table width, projection) -> GSADecodeStep, least recently used first
        self._max_fused_steps = 8
        # one native call per layer at decode; False keeps the separate operators (same results)
        self.fused_decode = bool(cfg.get("fused_decode", True))
        self.has_pc_hit = False
        self.prefix_block_ids = None      # int32 [sum of prefix blocks], all hit requests
        self.prefix_slot_mapping = None   # int64 [sum of prefix tokens]
        self._prefix_segments = []        # (first block, blocks, tokens) per hit request

    # ---- helpers mirroring the reference's names ----
    def get_layer_attn_metadata(self, forward_context, layer_name: str):
        attn_meta = forward_context.attn_metadata
        return attn_meta[layer_name] if isinstance(attn_meta, dict) else attn_meta

    def get_layer_state(self, layer_name: str):
        layer_id = int(layer_name.split(".")[2])
        return layer_id in self.hash_rollback_layers, False

    def hash_code(self, query: Optional[torch.Tensor] = None, nope: Optional[torch.Tensor] = None,
                  rope: Optional[torch.Tensor] = None, reduction_head_num: int = 1):
        """GQA: group-mean query -> one code per KV head (gsa_on_device.py:396-412).
        MLA: (nope codes, rope codes) of [T, H, D] or [T, D] inputs; with reduction_head_num > 1
        the H heads are first averaged down to H / reduction_head_num (:376-393)."""
        if self.is_mla:
            if nope is None or rope is None:
                raise ValueError("MLA mode requires `nope` and `rope`.")
            if reduction_head_num > 1:
                nope = nope.view(nope.shape[0], reduction_head_num, nope.shape[1] // reduction_head_num,
                                 nope.shape[2]).mean(dim=1)
                rope = rope.view(rope.shape[0], reduction_head_num, rope.shape[1] // reduction_head_num,
                                 rope.shape[2]).mean(dim=1)
            return (self.hash_encoder_nope.compute_hash(nope),
                    self.hash_encoder_rope.compute_hash(rope))
        if query is None:
            raise ValueError("GQA mode requires `query`.")
        if self.num_q_heads > self.num_key_heads:
            query = query.view(query.shape[0], self.num_key_heads,
                               self.num_q_heads // self.num_key_heads, query.shape[2]).mean(2)
        elif self.num_q_heads < self.num_key_heads:
            query = torch.repeat_interleave(query, self.num_key_heads // self.num_q_heads, dim=1)
        return self.hash_encoder.compute_hash(query)

    def rebuild_prefix_cache_info_for_req(self, block_table_row, num_prompt_tokens, qlen,
                                          block_size):
        """(num_prefix_tokens, num_prefix_blocks, prefix_block_ids, prefix_slot_mapping) of a
        request whose first num_prompt_tokens - qlen tokens came from the store
        (gsa_on_device.py:1142-1174)."""
        assert 0 <= qlen <= num_prompt_tokens
        num_prefix_tokens = num_prompt_tokens - qlen
        if num_prefix_tokens <= 0:
            empty = block_table_row[:0]
            return 0, 0, empty, empty
        num_prefix_blocks = (num_prefix_tokens + block_size - 1) // block_size
        prefix_block_ids = block_table_row[:num_prefix_blocks]
        token_idx = torch.arange(num_prefix_tokens, device=block_table_row.device)
        prefix_slot_mapping = (prefix_block_ids.index_select(0, token_idx // block_size).to(torch.int64)
                               * block_size + token_idx % block_size)
        return num_prefix_tokens, num_prefix_blocks, prefix_block_ids, prefix_slot_mapping

    def set_prefix_cache_hits(self, hits):
        """hits: iterable of (block_table_row, num_prompt_tokens, qlen) for the requests of this
        step whose prompt prefix was loaded from the store; sets has_pc_hit, prefix_block_ids
        and prefix_slot_mapping like build_sparse_meta (gsa_on_device.py:1322-1366)."""
        ids, slots, self._prefix_segments = [], [], []
        first = 0
        for row, num_prompt_tokens, qlen in hits:
            n_tok, n_blk, blk, slot = self.rebuild_prefix_cache_info_for_req(
                row, int(num_prompt_tokens), int(qlen), self.block_size)
            if n_tok > 0:
                ids.append(blk.to(torch.int32))
                slots.append(slot)
                self._prefix_segments.append((first, n_blk, n_tok))
                first += n_blk
        self.has_pc_hit = bool(ids)
        self.prefix_block_ids = torch.cat(ids) if ids else None
        self.prefix_slot_mapping = torch.cat(slots) if slots else None

    def cache_k_hash_gqa(self, key, attn_metadata, k_hash, k_cache=None):
        slots = attn_metadata.slot_mapping.flatten()
        n = slots.numel()
        self.hash_encoder.compute_hash_and_cache(
            key[:n].view(n, self.num_key_heads, self.head_dim), slots, k_hash,
            block_size=self.block_size)
        if self.has_pc_hit:
            # keys of the prefix are read where they lie in the paged KV cache (the reference
            # gathers them into a copy first, gsa_on_device.py:574-588)
            if k_cache is None:
                raise ValueError("a prefix-cache hit needs the layer's key cache")
            for first, n_blk, n_tok in self._prefix_segments:
                self.hash_encoder.compute_hash_from_paged_cache(
                    k_cache, self.prefix_block_ids[first:first + n_blk], n_tok, k_hash,
                    block_size=self.block_size)

    def _mla_code_views(self, k_hash):
        """The nope and rope byte ranges of a latent code cache [NB, BS, code] (any element type
        whose rows are (kv_lora_rank + qk_rope_head_dim) / 8 bytes) as rank-4 uint8 views."""
        u8 = k_hash if k_hash.dtype == torch.uint8 else k_hash.view(torch.uint8)
        if u8.ndim == 3:
            u8 = u8.unsqueeze(2)
        nb, rb = self.kv_lora_rank // 8, self.qk_rope_head_dim // 8
        if u8.ndim != 4 or u8.shape[2] != 1 or u8.shape[3] != nb + rb:
            raise ValueError(f"latent code cache must be [NB, BS, {nb + rb} bytes], got {tuple(k_hash.shape)}")
        return u8[..., :nb], u8[..., nb:]

    def cache_k_hash_mla(self, nope, rope, k_hash, attn_metadata, kv_cache=None):
        """Encode the step's latent keys and store the 18-word codes by slot
        (cache_k_hash_mla_cuda, gsa_on_device.py:426-455)."""
        slots = attn_metadata.slot_mapping.flatten()
        n = slots.numel()
        c_nope, c_rope = self._mla_code_views(k_hash)
        self.hash_encoder_nope.compute_hash_and_cache(
            nope[:n].reshape(n, 1, self.kv_lora_rank), slots, c_nope, block_size=self.block_size)
        self.hash_encoder_rope.compute_hash_and_cache(
            rope[:n].reshape(n, 1, self.qk_rope_head_dim), slots, c_rope, block_size=self.block_size)
        if self.has_pc_hit:
            self._rehash_prefix_mla(k_hash, kv_cache)

    def _rehash_prefix_mla(self, k_hash, kv_cache):
        """Codes of the prefix tokens that came from the store, read where their latents lie:
        kv_cache [NB, BS, kv_lora_rank + qk_rope_head_dim] (gsa_on_device.py:438-455)."""
        if kv_cache is None:
            raise ValueError("a prefix-cache hit needs the layer's latent cache")
        c_nope, c_rope = self._mla_code_views(k_hash)
        kc = kv_cache if kv_cache.ndim == 4 else kv_cache.unsqueeze(2)
        k_nope, k_rope = kc[..., :self.kv_lora_rank], kc[..., self.kv_lora_rank:]
        for first, n_blk, n_tok in self._prefix_segments:
            ids = self.prefix_block_ids[first:first + n_blk]
            self.hash_encoder_nope.compute_hash_from_paged_cache(k_nope, ids, n_tok, c_nope,
                                                                 block_size=self.block_size)
            self.hash_encoder_rope.compute_hash_from_paged_cache(k_rope, ids, n_tok, c_rope,
                                                                 block_size=self.block_size)

    def update_decode_topk_mla(self, layer_name, attn_metadata, decode_ql_nope, decode_q_pe, k_hash):
        """Top-k block table of a latent-attention decode step
        (update_decode_topk_mla_cuda, gsa_on_device.py:667-709)."""
        q_nope_hash, q_rope_hash = self.hash_code(nope=decode_ql_nope, rope=decode_q_pe,
                                                  reduction_head_num=self.hash_reduction_head_num)
        q_hash = torch.cat([q_nope_hash, q_rope_hash], dim=-1)
        u8 = k_hash if k_hash.dtype == torch.uint8 else k_hash.view(torch.uint8)
        meta = getattr(attn_metadata, "decode", attn_metadata)
        topk_table = cuda_hamming_topk(
            q_hash.unsqueeze(1), u8.unsqueeze(2) if u8.ndim == 3 else u8, meta.block_table,
            meta.seq_lens, topk_token=self.hash_topk_tokens, sink_token=self.block_size,
            recent_token=self.block_size * 4, is_mla=True)
        self._saved[layer_name] = (meta.block_table, meta.seq_lens)
        new_table = torch.zeros_like(meta.block_table)
        new_table[:, :topk_table.shape[1]] = topk_table
        new_lens = update_seq_lens(meta.seq_lens, self.hash_topk_tokens, self.block_size)
        if self.seq_len_threshold > 0:  # short requests keep their full table
            short = meta.seq_lens < self.seq_len_threshold
            new_table = torch.where(short[:, None], meta.block_table, new_table)
            new_lens = torch.where(short, meta.seq_lens, new_lens)
        meta.block_table = new_table
        meta.seq_lens = new_lens

    def _fused_decode_ok_mla(self, meta, k_hash, decode_ql_nope, decode_q_pe):
        """The single-call latent-attention step takes 16-bit inputs, int32 metadata, tables of at
        most 4096 blocks per request and a code cache [NB, BS, code] it can write in place as
        32-bit words; every other case runs the separate operators."""
        bt, sl = meta.block_table, meta.seq_lens
        code_bytes = (self.kv_lora_rank + self.qk_rope_head_dim) // 8
        return (self.fused_decode and self.dtype in (torch.bfloat16, torch.float16)
                and self.kv_lora_rank in (64, 128, 256, 512) and self.qk_rope_head_dim in (64, 128, 256, 512)
                and k_hash.dim() in (3, 4) and k_hash.is_contiguous()
                and k_hash.shape[-1] * k_hash.element_size() == code_bytes and code_bytes % 4 == 0
                and (k_hash.dim() == 3 or k_hash.shape[2] == 1)
                and decode_ql_nope is not None and decode_q_pe is not None
                and decode_ql_nope.dim() == 3 and decode_q_pe.dim() == 3
                and decode_ql_nope.stride(-1) == 1 and decode_q_pe.stride(-1) == 1
                and decode_ql_nope.shape[1] % self.hash_reduction_head_num == 0
                and bt.dtype == torch.int32 and sl.dtype == torch.int32 and bt.shape[1] <= 4096
                and bt.stride(-1) == 1 and sl.is_contiguous()
                and self.hash_topk_tokens % self.block_size == 0
                and self.hash_topk_tokens > 5 * self.block_size)

    def _fused_decode_step_mla(self, nope, rope, k_hash, attn_metadata, meta, decode_ql_nope, decode_q_pe,
                               kv_cache, layer_name):
        """cache_k_hash_mla + hash_code + cuda_hamming_topk + the table / length swap
        (gsa_on_device.py:426-455, 376-393, 667-709) as one native call."""
        bt, sl = meta.block_table, meta.seq_lens
        num_reqs = sl.shape[0]
        wn, wr = self.hash_encoder_nope.hash_weights, self.hash_encoder_rope.hash_weights
        hq = decode_ql_nope.shape[1]
        key_ = (num_reqs, bt.shape[1], hq, wn.data_ptr())
        step = self._fused_steps.pop(key_, None)  # re-inserted below: most recently used last
        if step is None:
            while len(self._fused_steps) >= self._max_fused_steps:  # each entry holds device buffers
                self._fused_steps.pop(next(iter(self._fused_steps)))
            step = GSADecodeStepMLA(wn, wr, hq, self.hash_reduction_head_num, num_reqs, bt.shape[1],
                                    self.hash_topk_tokens, block_size=self.block_size,
                                    sink_token=self.block_size, recent_token=4 * self.block_size,
                                    seq_len_threshold=self.seq_len_threshold)
        self._fused_steps[key_] = step
        slots = attn_metadata.slot_mapping.flatten()
        n = slots.numel()
        if self.has_pc_hit:  # prefix latents are re-encoded where they lie (gsa_on_device.py:438-455)
            self._rehash_prefix_mla(k_hash, kv_cache)
        words = k_hash.view(torch.int32)
        words = words.view(words.shape[0], words.shape[1], words.shape[-1])
        new_table, new_lens = step.step(nope[:n].reshape(n, self.kv_lora_rank),
                                        rope[:n].reshape(n, self.qk_rope_head_dim), slots,
                                        decode_ql_nope[:num_reqs], decode_q_pe[:num_reqs], words, bt, sl)
        self._saved[layer_name] = (bt, sl)
        meta.block_table = new_table
        meta.seq_lens = new_lens

    # ---- hooks ----
    def attention_begin(self, query, key, value, layer_name: str, forward_context, output=None,
                        phase: Optional[str] = None, k_hash=None, decode_ql_nope=None,
                        decode_q_pe=None):
        if not self.gsa_enabled or k_hash is None:
            return query, key, value, output
        attn_metadata = self.get_layer_attn_metadata(forward_context, layer_name)
        if self.is_mla:
            # key / value carry the latent vector and its rope part (gsa_on_device.py:872-880)
            kv_cache = None
            if self.has_pc_hit:
                attn = forward_context.no_compile_layers[layer_name]
                kv_cache = attn.kv_cache[forward_context.virtual_engine]
            is_rollback_layer, _ = self.get_layer_state(layer_name)
            decode = phase == "decode" and not is_rollback_layer
            meta = getattr(attn_metadata, "decode", attn_metadata)
            if decode and self._fused_decode_ok_mla(meta, k_hash, decode_ql_nope, decode_q_pe):
                self._fused_decode_step_mla(key, value, k_hash, attn_metadata, meta, decode_ql_nope,
                                            decode_q_pe, kv_cache, layer_name)
                return query, key, value, output
            self.cache_k_hash_mla(key, value, k_hash, attn_metadata, kv_cache)
            if decode:
                self.update_decode_topk_mla(layer_name, attn_metadata, decode_ql_nope, decode_q_pe,
                                            k_hash)
            return query, key, value, output
        k_cache = None
        if self.has_pc_hit:
            # kv_cache[0] is the key cache [NB, BS, Hkv, D] (gsa_on_device.py:576-579)
            attn = forward_context.no_compile_layers[layer_name]
            k_cache = attn.kv_cache[forward_context.virtual_engine][0]
        is_rollback_layer, _ = self.get_layer_state(layer_name)
        decode = phase == "decode" and not is_rollback_layer
        if decode and self._fused_decode_ok(attn_metadata, k_hash):
            self._fused_decode_step(query, key, attn_metadata, k_hash, k_cache, layer_name)
            return query, key, value, output
        self.cache_k_hash_gqa(key, attn_metadata, k_hash, k_cache)
        if decode:
            num_reqs = attn_metadata.seq_lens.shape[0]
            q = query[:num_reqs].view(num_reqs, self.num_q_heads, self.head_dim)
            q_hash = self.hash_code(q)
            topk_table = cuda_hamming_topk(
                q_hash.unsqueeze(1), k_hash, attn_metadata.block_table, attn_metadata.seq_lens,
                topk_token=self.hash_topk_tokens, sink_token=self.sink_tokens,
                recent_token=self.recent_tokens, is_mla=self.is_mla)
            self._saved[layer_name] = (attn_metadata.block_table, attn_metadata.seq_lens)
            topk = topk_table.shape[1]
            new_table = torch.zeros_like(attn_metadata.block_table)
            new_table[:, :topk] = topk_table
            new_lens = update_seq_lens(attn_metadata.seq_lens, self.hash_topk_tokens, self.block_size)
            if self.seq_len_threshold > 0:  # short requests keep their full table
                short = attn_metadata.seq_lens < self.seq_len_threshold
                new_table = torch.where(short[:, None], attn_metadata.block_table, new_table)
                new_lens = torch.where(short, attn_metadata.seq_lens, new_lens)
            attn_metadata.block_table = new_table
            attn_metadata.seq_lens = new_lens
        return query, key, value, output

    def _fused_decode_ok(self, attn_metadata, k_hash):
        """The single-call decode step takes 16-bit inputs with one projection, int32 metadata,
        tables of at most 4096 blocks per request and a code cache it can write in place (unit
        stride over a whole number of 32-bit words: anything else would be written into a copy);
        every other case runs the separate operators."""
        bt, sl = attn_metadata.block_table, attn_metadata.seq_lens
        return (self.fused_decode and self.dtype in (torch.bfloat16, torch.float16)
                and k_hash.stride(-1) == 1 and (k_hash.shape[-1] * k_hash.element_size()) % 4 == 0
                and self.head_dim in (64, 128, 256, 512) and self.hash_bits % 32 == 0
                and self.num_q_heads >= self.num_key_heads
                and bt.dtype == torch.int32 and sl.dtype == torch.int32 and bt.shape[1] <= 4096
                and bt.stride(-1) == 1 and sl.is_contiguous()
                and self.hash_topk_tokens % self.block_size == 0
                and self.recent_tokens > 0 and self.hash_topk_tokens > self.sink_tokens + self.recent_tokens)

    def _fused_decode_step(self, query, key, attn_metadata, k_hash, k_cache, layer_name):
        """cache_k_hash_gqa + hash_code + cuda_hamming_topk + the table / length swap of
        update_decode_topk_gqa_cuda (gsa_on_device.py:564-572, 773-811) as one native call."""
        bt, sl = attn_metadata.block_table, attn_metadata.seq_lens
        num_reqs = sl.shape[0]
        w = self.hash_encoder.hash_weights
        key_ = (num_reqs, bt.shape[1], w.data_ptr())
        step = self._fused_steps.pop(key_, None)  # re-inserted below: most recently used last
        if step is None:
            while len(self._fused_steps) >= self._max_fused_steps:  # each entry holds device buffers
                self._fused_steps.pop(next(iter(self._fused_steps)))
            step = GSADecodeStep(w, self.num_q_heads, self.num_key_heads, num_reqs,
                                 bt.shape[1], self.hash_topk_tokens, block_size=self.block_size,
                                 sink_token=self.sink_tokens, recent_token=self.recent_tokens,
                                 seq_len_threshold=self.seq_len_threshold)
        self._fused_steps[key_] = step
        slots = attn_metadata.slot_mapping.flatten()
        n = slots.numel()
        keys = key[:n].view(n, self.num_key_heads, self.head_dim)
        q = query[:num_reqs].view(num_reqs, self.num_q_heads, self.head_dim)
        if self.has_pc_hit:  # prefix keys are re-encoded where they lie (gsa_on_device.py:574-588)
            if k_cache is None:
                raise ValueError("a prefix-cache hit needs the layer's key cache")
            for first, n_blk, n_tok in self._prefix_segments:
                self.hash_encoder.compute_hash_from_paged_cache(
                    k_cache, self.prefix_block_ids[first:first + n_blk], n_tok, k_hash,
                    block_size=self.block_size)
        new_table, new_lens = step.step(keys, slots, q, _as_words(k_hash, "k_hash"), bt, sl)
        self._saved[layer_name] = (bt, sl)
        attn_metadata.block_table = new_table
        attn_metadata.seq_lens = new_lens

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context,
                           phase: Optional[str] = None) -> None:
        saved = self._saved.pop(layer_name, None)
        if saved is not None:
            attn_metadata = self.get_layer_attn_metadata(forward_context, layer_name)
            if self.is_mla:
                attn_metadata = getattr(attn_metadata, "decode", attn_metadata)
            attn_metadata.block_table, attn_metadata.seq_lens = saved

    def request_begin(self, request_id: Union[int, str], prompt_token_ids: List[int]):
        pass

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata):
        return GSAOnDeviceMetadata()
