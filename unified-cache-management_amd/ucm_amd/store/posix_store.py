"""The native posix store behind the reference's store interface.

`PosixStore` is the Python face of `ucm_posix_store_*` (csrc/posix_store.hip): one file per
block in the reference's on-disk format, so that a directory written by a UCM deployment can be
read here and the other way round.  Methods follow ucm/store/ucmstore_v1.py:41-204; config keys
are the reference's (ucm/store/posix/cc/posix_store.cc:104-129):

    storage_backends [dir, ...]      existing directories
    device_id                        >= 0 enables dump / load; -1 (default) is the lookup-only
                                     scheduler side, whose lookups refresh the files' mtime
    tensor_size, shard_size, block_size
    io_direct (False), timeout_ms (30000), data_dir_shard_bytes (3)
    posix_data_trans_concurrency     I/O threads per direction (default 16 here; the
                                     reference's default is 128)
    posix_lookup_concurrency (16)
    posix_io_engine                  "psync" (the only engine built; "aio" is rejected)
    posix_gc_enable (True), posix_capacity_gb (0 = no collection) or capacity_bytes,
    posix_gc_recycle_percent (0.1), posix_gc_trigger_threshold_ratio (0.7),
    posix_gc_shard_sample_ratio (0.1), posix_gc_max_recycle_count_per_shard (50000),
    posix_gc_check_interval_sec (30)

The store moves host memory: `dump` / `load` take CPU tensors, `dump_data` / `load_data` take
host addresses.  KV blocks in HBM reach it through a CacheStore in front (see pipeline.py).
"""
import ctypes as C
from typing import Dict, List

import numpy as np

from .. import _lib
from .base import Task, UcmKVStoreBaseV1
from .cache_store import CacheTask, _ids_array


class PosixStore(UcmKVStoreBaseV1):
    def __init__(self, config: Dict[str, object]) -> None:
        super().__init__(config)
        backends = config.get("storage_backends") or []
        if isinstance(backends, (str, bytes)):
            backends = [backends]
        engine = config.get("posix_io_engine", "psync")
        if engine != "psync":
            raise ValueError(f"invalid io engine({engine}): only psync is built")
        self._paths = [str(p).encode() for p in backends]
        arr = (C.c_char_p * max(len(self._paths), 1))(*self._paths)
        cfg = _lib.PosixConfig()
        cfg.storage_backends = C.cast(arr, C.POINTER(C.c_char_p))
        cfg.n_backends = len(self._paths)
        cfg.device_id = int(config.get("device_id", -1))
        cfg.io_direct = 1 if config.get("io_direct", False) else 0
        cfg.tensor_size = int(config.get("tensor_size", 0))
        cfg.shard_size = int(config.get("shard_size", 0))
        cfg.block_size = int(config.get("block_size", 0))
        cfg.data_trans_concurrency = int(config.get("posix_data_trans_concurrency", 16))
        cfg.lookup_concurrency = int(config.get("posix_lookup_concurrency", 16))
        cfg.timeout_ms = int(config.get("timeout_ms", 30000))
        cfg.data_dir_shard_bytes = int(config.get("data_dir_shard_bytes", 3))
        cfg.gc_enable = 1 if config.get("posix_gc_enable", True) else 0
        cap = config.get("capacity_bytes")
        if cap is None:
            cap = int(config.get("posix_capacity_gb", 0)) << 30
        cfg.capacity_bytes = int(cap)
        cfg.gc_recycle_percent = float(config.get("posix_gc_recycle_percent", 0.1))
        cfg.gc_trigger_threshold_ratio = float(config.get("posix_gc_trigger_threshold_ratio", 0.7))
        cfg.gc_shard_sample_ratio = float(config.get("posix_gc_shard_sample_ratio", 0.1))
        cfg.gc_max_recycle_count_per_shard = int(config.get("posix_gc_max_recycle_count_per_shard", 50000))
        cfg.gc_check_interval_sec = int(config.get("posix_gc_check_interval_sec", 30))
        self.tensor_size, self.shard_size, self.block_size = cfg.tensor_size, cfg.shard_size, cfg.block_size
        self.tensors_per_shard = cfg.shard_size // cfg.tensor_size if cfg.tensor_size else 0
        handle = C.c_void_p()
        _lib.check(_lib.lib().ucm_posix_store_create(C.byref(cfg), C.byref(handle)))
        self._h = handle

    def close(self):
        if getattr(self, "_h", None):
            _lib.check(_lib.lib().ucm_posix_store_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- layout ----
    def data_file_path(self, block_id: bytes, activated: bool = False) -> str:
        ids = _ids_array([block_id])
        buf = C.create_string_buffer(4096)
        n = _lib.lib().ucm_posix_store_data_file_path(self._h, ids.ctypes.data, 1 if activated else 0, buf, 4096)
        if n < 0:
            _lib.check(int(n))
        return buf.value.decode()

    def commit(self, block_id: bytes, success: bool = True) -> None:
        ids = _ids_array([block_id])
        _lib.check(_lib.lib().ucm_posix_store_commit(self._h, ids.ctypes.data, 1 if success else 0))

    def gc_once(self) -> int:
        removed = C.c_uint64(0)
        _lib.check(_lib.lib().ucm_posix_store_gc_once(self._h, C.byref(removed)))
        return int(removed.value)

    def native_backend(self, shard_size: int):
        """The C hooks that put this store beneath a CacheStore (which keeps a reference to
        this object, so the native store outlives it)."""
        if self.tensor_size != shard_size or self.shard_size != shard_size:
            raise ValueError(f"beneath a cache store tensor_size and shard_size must both be {shard_size}")
        cb = _lib.CacheBackend()
        _lib.check(_lib.lib().ucm_posix_store_backend(self._h, C.addressof(cb)))
        return cb

    # ---- interface ----
    def cc_store(self) -> int:
        return int(self._h.value)

    def lookup(self, block_ids: List[bytes]) -> List[bool]:
        ids = _ids_array(block_ids)
        found = np.zeros(len(block_ids), np.uint8)
        _lib.check(_lib.lib().ucm_posix_store_lookup(self._h, ids.ctypes.data, len(block_ids), found.ctypes.data))
        return [bool(v) for v in found]

    def lookup_on_prefix(self, block_ids: List[bytes]) -> int:
        ids = _ids_array(block_ids)
        last = C.c_int64(-1)
        _lib.check(_lib.lib().ucm_posix_store_lookup_on_prefix(self._h, ids.ctypes.data, len(block_ids),
                                                               C.byref(last)))
        return int(last.value)

    def prefetch(self, block_ids: List[bytes]) -> None:
        return None  # posix_store.cc:74: a no-op in the reference too

    def _submit(self, load, block_ids, shard_index, addrs):
        n = len(block_ids)
        if len(shard_index) != n:
            raise ValueError("block_ids and shard_index differ in length")
        ids = _ids_array(block_ids)
        idx = np.ascontiguousarray(np.asarray(shard_index, dtype=np.uint64))
        a = np.ascontiguousarray(np.asarray(addrs, dtype=np.uint64)).reshape(n, -1) if n else np.zeros((0, 1), np.uint64)
        if n and self.tensors_per_shard and a.shape[1] != self.tensors_per_shard:
            raise ValueError(f"addresses must be [{n}, {self.tensors_per_shard}], got {a.shape}")
        task = C.c_int64(0)
        fn = _lib.lib().ucm_posix_store_load if load else _lib.lib().ucm_posix_store_dump
        _lib.check(fn(self._h, ids.ctypes.data, idx.ctypes.data, a.ctypes.data, n, C.byref(task)))
        return CacheTask(int(task.value))

    def load_data(self, block_ids, shard_index, dst_addr) -> Task:
        return self._submit(True, block_ids, shard_index, dst_addr)

    def dump_data(self, block_ids, shard_index, src_addr, prerequisite_handle: int = 0) -> Task:
        if prerequisite_handle:
            raise ValueError("the posix store moves host memory and takes no device event")
        return self._submit(False, block_ids, shard_index, src_addr)

    def _tensor_rows(self, tensors, n):
        rows = []
        for row in tensors:
            for t in row:
                if t.device.type != "cpu":
                    raise ValueError("the posix store moves host memory: put a CacheStore in front for GPU tensors")
            rows.append([int(t.data_ptr()) for t in row])
        if len(rows) != n:
            raise ValueError("one row of tensors per block expected")
        return rows

    def load(self, block_ids, shard_index, dst_tensor) -> Task:
        return self.load_data(block_ids, shard_index, self._tensor_rows(dst_tensor, len(block_ids)))

    def dump(self, block_ids, shard_index, src_tensor) -> Task:
        return self.dump_data(block_ids, shard_index, self._tensor_rows(src_tensor, len(block_ids)))

    def wait(self, task: Task) -> None:
        _lib.check(_lib.lib().ucm_posix_store_wait(self._h, task.task_id))

    def check(self, task: Task) -> bool:
        fin = C.c_int32(0)
        _lib.check(_lib.lib().ucm_posix_store_check(self._h, task.task_id, C.byref(fin)))
        return bool(fin.value)
