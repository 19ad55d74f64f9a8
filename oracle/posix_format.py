"""The posix store's on-disk format restated in Python — TEST INFRASTRUCTURE ONLY.

Follows ucm/store/posix/cc/space_layout.cc:53-56 (file name), :88-99 (path), :101-111 (commit
by rename), :164-170 (backend choice) and trans_queue.cc:127-169 (where a shard's bytes sit in
the file).  The reference's implementation cannot be compiled here (its sources include the
project logger, which needs spdlog; the image has none), so this restatement is pinned by the
expectations written in the reference's own tests
(ucm/store/test/case/posix/posix_space_manager_test.cc:64-111: "<backend>data/<hex>.tmp",
"<backend>data/<hex>", "<backend><first n digits>/<hex>[.tmp]") — see tests/test_posix_format.py.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_HASH = None


def block_id_hash(block_id: bytes) -> int:
    """std::hash<std::string_view> of the 16 id bytes, from the C++ standard library."""
    global _HASH
    if _HASH is None:
        so = os.path.join(_HERE, "libucm_oracle_hash.so")
        if not os.path.exists(so):
            from . import c_api
            c_api.build(force=True)
        _HASH = C.CDLL(so)
        _HASH.oracle_block_id_hash.restype = C.c_uint64
        _HASH.oracle_block_id_hash.argtypes = [C.c_char_p]
    assert len(block_id) == 16
    return int(_HASH.oracle_block_id_hash(bytes(block_id)))


def file_name(block_id: bytes) -> str:
    return "".join(f"{b:02x}" for b in block_id)


def data_file_path(backends, block_id: bytes, activated: bool, shard_digits: int) -> str:
    backends = [b if b.endswith("/") else b + "/" for b in backends]
    backend = backends[0] if len(backends) == 1 else backends[block_id_hash(block_id) % len(backends)]
    name = file_name(block_id)
    directory = name[:shard_digits] if shard_digits > 0 else "data"
    return f"{backend}{directory}/{name}" + (".tmp" if activated else "")


def write_block(backends, block_id: bytes, shards, shard_size: int, shard_digits: int, commit=True):
    """Writes a block file as the reference's dump does: every shard (a list of equally sized
    byte strings, its tensors) at offset index * shard_size under the .tmp name, then the
    rename.  `shards` maps shard index -> list of tensors."""
    tmp = data_file_path(backends, block_id, True, shard_digits)
    os.makedirs(os.path.dirname(tmp), exist_ok=True)
    with open(tmp, "wb") as f:
        for index, tensors in shards.items():
            off = index * shard_size
            for t in tensors:
                f.seek(off)
                f.write(t)
                off += len(t)
    if commit:
        os.rename(tmp, data_file_path(backends, block_id, False, shard_digits))


def read_shard(backends, block_id: bytes, index: int, shard_size: int, tensor_size: int, shard_digits: int):
    path = data_file_path(backends, block_id, False, shard_digits)
    with open(path, "rb") as f:
        f.seek(index * shard_size)
        raw = f.read(shard_size)
    return [raw[o:o + tensor_size] for o in range(0, shard_size, tensor_size)]
