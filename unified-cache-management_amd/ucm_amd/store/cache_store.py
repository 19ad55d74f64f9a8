"""The native cache store behind the reference's store interface.

`CacheStore` is the Python face of `ucm_cache_store_*` (csrc/cache_store.hip): a pinned-host
staging cache with dump and load worker threads, in front of an optional slower backend — what
`UcmCacheStore` is to the reference's C++ CacheStore (ucm/store/cache/connector.py over
ucm/store/cache/cc/).  Methods and argument meaning follow ucm/store/ucmstore_v1.py:41-204.

config keys (names from cache_store.cc:104-131 where they exist):
    tensor_size_list [bytes per tensor of a shard ...]  or  tensor_size + shard_size
    cache_buffer_capacity_gb  or  buffer_capacity_bytes     pinned staging memory
    device_id (default 0), waiting_queue_depth (default 8192), timeout_ms (default 30000)
    store_backend: optional; either a PosixStore (chained natively through its C hooks) or any
        object with lookup(ids) -> [bool], dump(ids, shard_idx, views) and
        load(ids, shard_idx, views); `views` are writable uint8 numpy views of the pinned
        shards.  It stands where the reference passes the next StoreV1*.
"""
import ctypes as C
import threading
from typing import Dict, List

import numpy as np

from .. import _lib
from .base import Task, UcmKVStoreBaseV1


_Backend = _lib.CacheBackend


def _ids_array(block_ids: List[bytes]) -> np.ndarray:
    out = np.zeros((len(block_ids), 16), np.uint8)
    for i, b in enumerate(block_ids):
        b = bytes(b)
        if len(b) != 16:
            raise ValueError(f"block id {i} has {len(b)} bytes, expected 16")
        out[i] = np.frombuffer(b, np.uint8)
    return out


class CacheTask(Task):
    def __init__(self, task_id: int):
        self.task_id = task_id


class CacheStore(UcmKVStoreBaseV1):
    def __init__(self, config: Dict[str, object]) -> None:
        super().__init__(config)
        sizes = config.get("tensor_size_list")
        if sizes is None:
            tensor_size, shard_size = int(config["tensor_size"]), int(config["shard_size"])
            if tensor_size <= 0 or shard_size % tensor_size:
                raise ValueError(f"invalid shard size({shard_size})")
            sizes = [tensor_size] * (shard_size // tensor_size)
        self.tensor_sizes = np.asarray(sizes, dtype=np.uint64).reshape(-1)
        if self.tensor_sizes.size == 0 or not np.all(self.tensor_sizes > 0):
            raise ValueError("invalid tensor size")
        self.shard_size = int(self.tensor_sizes.sum())
        cap = config.get("buffer_capacity_bytes")
        if cap is None:
            cap = int(config.get("cache_buffer_capacity_gb", 1)) << 30
        self._py_backend = config.get("store_backend")
        self._cb = None
        backend_ptr = None
        if hasattr(self._py_backend, "native_backend"):
            # a native store (the posix store): its own C hooks, no Python in the data path
            self._cb = self._py_backend.native_backend(self.shard_size)
            backend_ptr = C.addressof(self._cb)
        elif self._py_backend is not None:
            self._cb = self._make_callbacks(self._py_backend)
            backend_ptr = C.addressof(self._cb)
        handle = C.c_void_p()
        arr = (C.c_size_t * self.tensor_sizes.size)(*[int(v) for v in self.tensor_sizes])
        _lib.check(_lib.lib().ucm_cache_store_create(
            int(config.get("device_id", 0)), arr, self.tensor_sizes.size, int(cap),
            int(config.get("waiting_queue_depth", 8192)), int(config.get("timeout_ms", 30000)),
            backend_ptr, C.byref(handle)))
        self._h = handle

    # ---- backend trampolines: the native threads call back into Python ----
    def _make_callbacks(self, be):
        shard = self.shard_size
        lock = threading.Lock()
        state = {"next": 1}

        def views(host_ptrs, n):
            ptrs = np.ctypeslib.as_array(C.cast(host_ptrs, C.POINTER(C.c_uint64)), shape=(n,))
            return [np.ctypeslib.as_array(C.cast(int(p), C.POINTER(C.c_uint8)), shape=(shard,))
                    for p in ptrs]

        def ids_of(ptr, n):
            raw = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(n, 16))
            return [bytes(r) for r in raw]

        def idx_of(ptr, n):
            return [int(v) for v in np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint64)), shape=(n,))]

        def lookup(_ctx, ids, n, found):
            try:
                res = be.lookup(ids_of(ids, n))
                out = np.ctypeslib.as_array(C.cast(found, C.POINTER(C.c_uint8)), shape=(n,))
                out[:] = np.asarray(res, dtype=np.uint8)
                return 0
            except Exception:
                return -1

        def mover(fn):
            def call(_ctx, ids, idx, host, n, _shard):
                try:
                    fn(ids_of(ids, n), idx_of(idx, n), views(host, n))
                    with lock:
                        h = state["next"]
                        state["next"] += 1
                    return h
                except Exception:
                    return -1
            return call

        cb = _Backend()
        cb.ctx = None
        cb.lookup = _Backend.LOOKUP(lookup)
        cb.dump = _Backend.MOVE(mover(be.dump))
        cb.load = _Backend.MOVE(mover(be.load))
        cb.wait = _Backend.WAIT(lambda _ctx, _h: 0)  # the Python hooks are synchronous
        return cb

    def close(self):
        if getattr(self, "_h", None):
            _lib.check(_lib.lib().ucm_cache_store_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- interface ----
    def cc_store(self) -> int:
        return int(self._h.value)

    @property
    def nodes(self) -> int:
        return int(_lib.lib().ucm_cache_store_nodes(self._h))

    def lookup(self, block_ids: List[bytes]) -> List[bool]:
        ids = _ids_array(block_ids)
        found = np.zeros(len(block_ids), np.uint8)
        _lib.check(_lib.lib().ucm_cache_store_lookup(self._h, ids.ctypes.data, len(block_ids),
                                                     found.ctypes.data))
        return [bool(v) for v in found]

    def lookup_on_prefix(self, block_ids: List[bytes]) -> int:
        ids = _ids_array(block_ids)
        last = C.c_int64(-1)
        _lib.check(_lib.lib().ucm_cache_store_lookup_on_prefix(self._h, ids.ctypes.data,
                                                               len(block_ids), C.byref(last)))
        return int(last.value)

    def prefetch(self, block_ids: List[bytes]) -> None:
        return None  # a hint the reference's cache store ignores as well (cache_store.cc:71)

    def _addr_rows(self, addrs, n):
        a = np.ascontiguousarray(np.asarray(addrs, dtype=np.uint64))
        if a.shape != (n, self.tensor_sizes.size):
            raise ValueError(f"addresses must be [{n}, {self.tensor_sizes.size}], got {a.shape}")
        return a

    def _submit(self, load, block_ids, shard_index, addrs, prerequisite_handle=0):
        n = len(block_ids)
        if len(shard_index) != n:
            raise ValueError("block_ids and shard_index differ in length")
        ids = _ids_array(block_ids)
        idx = np.ascontiguousarray(np.asarray(shard_index, dtype=np.uint64))
        a = self._addr_rows(addrs, n)
        task = C.c_int64(0)
        if load:
            _lib.check(_lib.lib().ucm_cache_store_load(self._h, ids.ctypes.data, idx.ctypes.data,
                                                       a.ctypes.data, n, C.byref(task)))
        else:
            _lib.check(_lib.lib().ucm_cache_store_dump(self._h, ids.ctypes.data, idx.ctypes.data,
                                                       a.ctypes.data, n,
                                                       int(prerequisite_handle) or None, C.byref(task)))
        return CacheTask(int(task.value))

    def load_data(self, block_ids, shard_index, dst_addr) -> Task:
        return self._submit(True, block_ids, shard_index, dst_addr)

    def dump_data(self, block_ids, shard_index, src_addr, prerequisite_handle: int = 0) -> Task:
        return self._submit(False, block_ids, shard_index, src_addr, prerequisite_handle)

    def _tensor_rows(self, tensors, n):
        # one row of tensors per block, as ucmstore_v1.py's load/dump take them
        rows = [[int(t.data_ptr()) for t in row] for row in tensors]
        if len(rows) != n:
            raise ValueError("one row of tensors per block expected")
        return rows

    def load(self, block_ids, shard_index, dst_tensor) -> Task:
        return self.load_data(block_ids, shard_index, self._tensor_rows(dst_tensor, len(block_ids)))

    def dump(self, block_ids, shard_index, src_tensor) -> Task:
        return self.dump_data(block_ids, shard_index, self._tensor_rows(src_tensor, len(block_ids)))

    def wait(self, task: Task) -> None:
        _lib.check(_lib.lib().ucm_cache_store_wait(self._h, task.task_id))

    def check(self, task: Task) -> bool:
        fin = C.c_int(0)
        _lib.check(_lib.lib().ucm_cache_store_check(self._h, task.task_id, C.byref(fin)))
        return bool(fin.value)
