"""HashEncoder: float tensor -> packed sign-hash codes, on MI355X.

Host-side mirror of the reference's HashEncoder
(ucm/sparse/gsa_on_device/hash_encoder.py:373-662): same constructor, same method names,
same argument meaning and the same ValueError behaviour on shape / device / dtype
mismatches.  The arithmetic runs in libucm_hip.so (MFMA for bf16 / fp16, FMA for fp32).

Extension over the reference: one projection matrix per group of heads
(`set_hash_weight` accepts [n_w, input_dim, hash_bits]; head h uses matrix
min(h // heads_per_weight, n_w - 1)).
"""
import torch

from .. import _lib

_DT = {torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16, torch.float32: _lib.DT_F32}


class HashEncoder:
    """Converts a float tensor to a binary hash code tensor, 8 bits per uint8, LSB first."""

    def __init__(self, input_dim: int, hash_bits: int, dtype: torch.dtype, device: torch.device,
                 num_weights: int = 1, heads_per_weight: int = 1) -> None:
        self.input_dim = input_dim
        if hash_bits % 8 != 0:
            raise ValueError("hash_bits must be a multiple of 8")
        self.hash_bits = hash_bits
        self.hash_numbers = hash_bits // 8
        if dtype not in _DT:
            raise ValueError(f"unsupported dtype {dtype}; use bfloat16, float16 or float32")
        self.dtype = dtype
        self.device = torch.device(device)
        self.num_weights = int(num_weights)
        self.heads_per_weight = int(heads_per_weight)
        # the kernels produce whole 32-bit words; extra columns are zero and give 0 bits
        self._padded_bits = (hash_bits + 31) // 32 * 32
        self._init_hash_weights()
        self._init_bit_masks()

    # -- weights ------------------------------------------------------------------------
    def _init_hash_weights(self):
        # Gaussian(std 2) -> QR -> Q * sign(diag R): Haar-distributed orthogonal columns
        # (hash_encoder.py:412-425).  Done in fp32 on the host; only the result is cast.
        ws = []
        for _ in range(self.num_weights):
            g = torch.normal(mean=0.0, std=2.0, size=(self.input_dim, self.hash_bits),
                             dtype=torch.float32)
            q, r = torch.linalg.qr(g)
            ws.append(q * torch.sign(torch.diag(r)))
        w = torch.stack(ws) if self.num_weights > 1 else ws[0]
        self.hash_weights = w.to(self.dtype).to(self.device)
        self._refresh_padded()

    def _refresh_padded(self):
        w = self.hash_weights
        w3 = w if w.dim() == 3 else w.unsqueeze(0)
        if self._padded_bits != self.hash_bits:
            pad = torch.zeros(w3.shape[0], self.input_dim, self._padded_bits - self.hash_bits,
                              dtype=w3.dtype, device=w3.device)
            w3 = torch.cat([w3, pad], dim=-1)
        self._w = w3.contiguous()

    def set_hash_weight(self, hash_weights: torch.Tensor) -> None:
        ok2 = tuple(hash_weights.shape) == (self.input_dim, self.hash_bits) and self.num_weights == 1
        ok3 = tuple(hash_weights.shape) == (self.num_weights, self.input_dim, self.hash_bits)
        if not (ok2 or ok3):
            raise ValueError(
                f"hash_weights shape {tuple(hash_weights.shape)} does not match required shape "
                f"{(self.input_dim, self.hash_bits)}")
        if hash_weights.dtype != self.dtype:
            raise ValueError(
                f"hash_weights dtype {hash_weights.dtype} does not match required dtype {self.dtype}")
        if hash_weights.device != self.hash_weights.device:
            raise ValueError(
                f"hash_weights device {hash_weights.device} does not match required device "
                f"{self.device}")
        self.hash_weights = hash_weights.clone()
        self._refresh_padded()

    def _init_bit_masks(self) -> None:
        self.bit_masks = torch.pow(2, torch.arange(8, dtype=torch.uint8, device=self.device))

    # -- helpers ------------------------------------------------------------------------
    def _check_x(self, x):
        if x.shape[-1] != self.input_dim:
            raise ValueError(f"x must be of shape (..., {self.input_dim}), but got {x.shape}")
        if x.device != self.hash_weights.device:
            raise ValueError(f"x device {x.device} does not match required device {self.device}")
        if x.device.type != "cuda":
            raise ValueError("the HIP library needs tensors on a GPU device")

    def _prep(self, x):
        if x.dtype != self.dtype:
            x = x.to(self.dtype)
        if x.stride(-1) != 1:
            x = x.contiguous()
        return x

    # -- operators ----------------------------------------------------------------------
    def compute_hash(self, x: torch.Tensor, per_head: bool = False) -> torch.Tensor:
        """x (..., input_dim) -> uint8 (..., hash_bits // 8).

        per_head=False: one matrix for all rows (the reference's behaviour).
        per_head=True : x is (..., H, input_dim); head h is projected with matrix
                        min(h // heads_per_weight, num_weights - 1).
        """
        self._check_x(x)
        orig_shape = x.shape[:-1]
        x = self._prep(x)
        if per_head:
            H = x.shape[-2]
            x3 = x.reshape(-1, H, self.input_dim)
            hpw = self.heads_per_weight
        else:
            H = 1
            x3 = x.reshape(-1, 1, self.input_dim)
            hpw = 0
        T = x3.shape[0]
        Wd = self._padded_bits // 32
        out = torch.empty((T, H, Wd), dtype=torch.int32, device=x.device)
        if T > 0:
            _lib.check(_lib.lib().ucm_hash_encode(
                x3.data_ptr(), _DT[self.dtype], T, H, self.input_dim, _lib.stride(x3, 0),
                _lib.stride(x3, 1),
                self._w.data_ptr(), _DT[self.dtype], self._w.shape[0], hpw, self._padded_bits,
                out.data_ptr(), _lib.stride(out, 0), _lib.stride(out, 1), _lib.stream_ptr(x.device)))
        codes = out.view(torch.uint8)[..., : self.hash_numbers]
        return codes.reshape(*orig_shape, self.hash_numbers)

    def _reinterpret_cache_as_u8(self, cache: torch.Tensor) -> torch.Tensor:
        # uint8 [..., hash_numbers] or a wider element type viewed as bytes
        # (hash_encoder.py:509-546 accepts uint8 and bfloat16)
        if cache.dtype == torch.uint8:
            u8 = cache
        elif cache.dtype in (torch.bfloat16, torch.float16, torch.int16, torch.int32, torch.float32):
            if (self.hash_numbers % cache.element_size()) != 0:
                raise ValueError(
                    f"for {cache.dtype} cache, hash_numbers must be a multiple of "
                    f"{cache.element_size()}, got {self.hash_numbers}")
            u8 = cache.view(torch.uint8)
        else:
            raise ValueError(f"unsupported k_hash_cache dtype {cache.dtype}")
        if u8.shape[-1] != self.hash_numbers:
            raise ValueError(
                f"cache last dim mismatch: got {u8.shape[-1]} bytes, expected {self.hash_numbers}")
        return u8

    def compute_hash_and_cache(self, x: torch.Tensor, slot_mapping: torch.Tensor,
                               k_hash_cache: torch.Tensor, block_size: int = 128,
                               **_tuning) -> torch.Tensor:
        """Encode x [T,H,K] and store each code at k_hash_cache[slot // BS, slot % BS, h, :].
        Slots < 0 or >= NB*BS are skipped.  Returns k_hash_cache.  Tile-size keyword arguments
        of the reference's Triton launcher are accepted and ignored."""
        if x.ndim != 3:
            raise ValueError(f"x must be [T,H,K], got {x.shape}")
        if slot_mapping.ndim != 1:
            raise ValueError(f"slot_mapping must be [T], got {slot_mapping.shape}")
        if k_hash_cache.ndim != 4:
            raise ValueError(f"k_hash_cache must be rank-4, got {k_hash_cache.shape}")
        self._check_x(x)
        if slot_mapping.device != x.device:
            raise ValueError(
                f"slot_mapping device {slot_mapping.device} does not match required device {self.device}")
        if k_hash_cache.device != x.device:
            raise ValueError(
                f"k_hash_cache device {k_hash_cache.device} does not match required device {self.device}")
        T, H, _ = x.shape
        NB, BS, H_cache, _ = k_hash_cache.shape
        if slot_mapping.shape[0] != T:
            raise ValueError(f"slot_mapping length {slot_mapping.shape[0]} != T {T}")
        if BS != block_size:
            raise ValueError(f"k_hash_cache.shape[1]={BS} != block_size={block_size}")
        if H_cache != H:
            raise ValueError(f"k_hash_cache.shape[2]={H_cache} != H={H}")
        if self.hash_bits % 32 != 0:
            raise NotImplementedError("the fused cache write needs hash_bits % 32 == 0")
        u8 = self._reinterpret_cache_as_u8(k_hash_cache)
        sb, ss, sh, sw = (_lib.stride(u8, d) for d in range(4))
        if sw != 1 or sb % 4 or ss % 4 or sh % 4 or u8.data_ptr() % 4:
            raise ValueError("k_hash_cache codes must be contiguous and 4-byte aligned")
        if slot_mapping.dtype not in (torch.int32, torch.int64):
            raise ValueError(f"slot_mapping dtype {slot_mapping.dtype} must be int32 or int64")
        slot_mapping = slot_mapping.contiguous()
        x = self._prep(x)
        if T > 0:
            _lib.check(_lib.lib().ucm_hash_encode_cache(
                x.data_ptr(), _DT[self.dtype], T, H, self.input_dim, _lib.stride(x, 0),
                _lib.stride(x, 1),
                self._w.data_ptr(), _DT[self.dtype], self._w.shape[0],
                self.heads_per_weight if self.num_weights > 1 else 0, self._padded_bits,
                slot_mapping.data_ptr(), int(slot_mapping.dtype == torch.int64),
                u8.data_ptr(), NB, BS, sb // 4, ss // 4, sh // 4, _lib.stream_ptr(x.device)))
        return k_hash_cache

    def compute_hash_from_paged_cache(self, k_cache: torch.Tensor, block_ids: torch.Tensor,
                                      num_tokens: int, k_hash_cache: torch.Tensor,
                                      block_size: int = 128) -> torch.Tensor:
        """Prefix-cache rehash: encode the first `num_tokens` tokens of the key blocks
        `block_ids` of the paged KV cache k_cache [NB,BS,H,K] in place and store each code at
        the same block and token of k_hash_cache [NB',BS,H,W].

        One call for what the reference does with a gathered copy
        (`kv_cache[0][0][prefix_block_ids]`, reshape, compute_hash_and_cache with the prefix
        slot mapping, gsa_on_device.py:574-588); slot(i) = block_ids[i // BS] * BS + i % BS
        as in rebuild_prefix_cache_info_for_req (:1142-1174).  Returns k_hash_cache."""
        if k_cache.ndim != 4:
            raise ValueError(f"k_cache must be [NB,BS,H,K], got {k_cache.shape}")
        if k_hash_cache.ndim != 4:
            raise ValueError(f"k_hash_cache must be rank-4, got {k_hash_cache.shape}")
        if block_ids.ndim != 1 or block_ids.dtype != torch.int32:
            raise ValueError("block_ids must be int32 [n_blocks]")
        self._check_x(k_cache)
        if block_ids.device != k_cache.device or k_hash_cache.device != k_cache.device:
            raise ValueError(f"all tensors must be on {self.device}")
        if k_cache.dtype != self.dtype:
            raise ValueError(f"k_cache dtype {k_cache.dtype} != encoder dtype {self.dtype}")
        NBk, BS, H, _ = k_cache.shape
        NB, BSc, Hc, _ = k_hash_cache.shape
        if BS != block_size or BSc != block_size:
            raise ValueError(f"block sizes {BS}, {BSc} != block_size={block_size}")
        if Hc != H:
            raise ValueError(f"k_hash_cache.shape[2]={Hc} != H={H}")
        n_blocks = int(block_ids.shape[0])
        num_tokens = int(num_tokens)
        if num_tokens < 0 or num_tokens > n_blocks * BS:
            raise ValueError(f"num_tokens {num_tokens} does not fit {n_blocks} blocks of {BS}")
        if self.hash_bits % 32 != 0:
            raise NotImplementedError("the fused cache write needs hash_bits % 32 == 0")
        if k_cache.stride(-1) != 1:
            raise ValueError("the K values of a row must be contiguous")
        u8 = self._reinterpret_cache_as_u8(k_hash_cache)
        sb, ss, sh, sw = (_lib.stride(u8, d) for d in range(4))
        if sw != 1 or sb % 4 or ss % 4 or sh % 4 or u8.data_ptr() % 4:
            raise ValueError("k_hash_cache codes must be contiguous and 4-byte aligned")
        block_ids = block_ids.contiguous()
        if num_tokens > 0:
            _lib.check(_lib.lib().ucm_hash_encode_paged(
                k_cache.data_ptr(), _DT[self.dtype], NBk, BS, H, self.input_dim,
                _lib.stride(k_cache, 0), _lib.stride(k_cache, 1), _lib.stride(k_cache, 2),
                block_ids.data_ptr(), n_blocks, num_tokens,
                self._w.data_ptr(), _DT[self.dtype], self._w.shape[0],
                self.heads_per_weight if self.num_weights > 1 else 0, self._padded_bits,
                u8.data_ptr(), NB, sb // 4, ss // 4, sh // 4, _lib.stream_ptr(k_cache.device)))
        return k_hash_cache

    def reshape_and_cache(self, k_hash_compute: torch.Tensor, slot_mapping: torch.Tensor,
                          k_hash: torch.Tensor, block_size: int = 128) -> torch.Tensor:
        """Scatter precomputed codes [T,H,W] into the paged cache [NB,BS,H,W]
        (reshape_and_cache_khash_triton, hash_encoder.py:197-261)."""
        return reshape_and_cache_khash(k_hash_compute, slot_mapping, k_hash, block_size)

    def _unpack_hash(self, packed_codes: torch.Tensor) -> torch.Tensor:
        """uint8 (..., hash_numbers) -> float16 (..., hash_bits) of +-1 (hash_encoder.py:664-726)."""
        if packed_codes.shape[-1] != self.hash_numbers:
            raise ValueError(
                f"packed_codes must be of shape (..., {self.hash_numbers}), but got {packed_codes.shape}")
        if packed_codes.dtype != torch.uint8:
            raise ValueError(f"packed_codes dtype {packed_codes.dtype} is not torch.uint8")
        masks = self.bit_masks.to(packed_codes.device)
        bits = (packed_codes.unsqueeze(-1) & masks) > 0
        return (bits.to(torch.float16) * 2 - 1).reshape(*packed_codes.shape[:-1], self.hash_bits)


def reshape_and_cache_khash(k_hash_compute, slot_mapping, k_hash, block_size=128):
    """Scatter codes [T,H,W] (any 1/2/4-byte element type) into k_hash [NB,BS,H,W] by slot."""
    if k_hash_compute.ndim != 3:
        raise ValueError(f"expect [T,H,W], got {k_hash_compute.shape}")
    if k_hash.ndim != 4:
        raise ValueError(f"expect [B,BS,H,W], got {k_hash.shape}")
    if slot_mapping.ndim != 1 or slot_mapping.shape[0] != k_hash_compute.shape[0]:
        raise ValueError("slot_mapping must be [T]")
    if k_hash.shape[1] != block_size:
        raise ValueError(f"k_hash BS={k_hash.shape[1]} != block_size={block_size}")
    if tuple(k_hash_compute.shape[1:]) != tuple(k_hash.shape[2:]) or k_hash_compute.dtype != k_hash.dtype:
        raise ValueError(
            f"shape mismatch: compute {k_hash_compute.shape[1:]} vs cache {k_hash.shape[2:]}")
    src = k_hash_compute.contiguous().view(torch.uint8)
    dst = k_hash.view(torch.uint8)
    T, H, Wb = src.shape
    sb, ss, sh, sw = (_lib.stride(dst, d) for d in range(4))
    if Wb % 4 or sw != 1 or sb % 4 or ss % 4 or sh % 4:
        raise ValueError("codes must be a whole number of 4-byte words and 4-byte aligned")
    slot_mapping = slot_mapping.contiguous()
    if T > 0:
        _lib.check(_lib.lib().ucm_code_scatter(
            src.data_ptr(), T, H, Wb // 4, _lib.stride(src, 0) // 4, _lib.stride(src, 1) // 4,
            slot_mapping.data_ptr(), int(slot_mapping.dtype == torch.int64), dst.data_ptr(),
            k_hash.shape[0], block_size, sb // 4, ss // 4, sh // 4,
            _lib.stream_ptr(k_hash.device)))
    return k_hash
