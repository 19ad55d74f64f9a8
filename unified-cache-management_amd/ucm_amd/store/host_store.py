"""A host-memory KV store on top of the MI355X transfer path.

Implements the reference's store interface (ucm/store/ucmstore_v1.py:41-204) with pinned host
memory as the only tier, so that the gather/scatter kernels are reachable exactly the way the
connector reaches a UCM store: `dump_data(block_ids, shard_index, src_addr, event)` gathers the
device chunks of each block into one pinned slot (what CacheStore's dump queue does with its
staging buffer, ucm/store/cache/cc/dump_queue.cc:91-161) and `load_data` scatters a slot back
(load_queue.cc:128-194).  No file back-end, no eviction: a full store raises.

config: {"tensor_size_list": [bytes per pointer column ...] or "tensor_size": int,
         "capacity_blocks": int, "device_id": int (default 0), "stream_number": int (default 1)}
"""
import threading
from typing import Dict, List

import numpy as np

from ..trans import Device, host_view
from .base import Task, UcmKVStoreBaseV1


class _Task(Task):
    def __init__(self):
        self.done = threading.Event()
        self.ok = True


class HostMemoryStore(UcmKVStoreBaseV1):
    def __init__(self, config: Dict[str, object]) -> None:
        super().__init__(config)
        sizes = config.get("tensor_size_list")
        if sizes is None:
            sizes = [int(config["tensor_size"])]
        self.sizes = np.asarray(sizes, dtype=np.uint64).reshape(-1)
        self.uniform = bool(np.all(self.sizes == self.sizes[0]))
        self.slot_bytes = int(self.sizes.sum())
        self.capacity = int(config["capacity_blocks"])
        self.device = Device()
        self.device.Setup(int(config.get("device_id", 0)))
        self.buffer = self.device.MakeBuffer()
        self.slab = self.buffer.MakeHostBuffer(self.slot_bytes * self.capacity)
        n_streams = max(1, int(config.get("stream_number", 1)))
        self.streams = [self.device.MakeSMStream() for _ in range(n_streams)]
        self._rr = 0
        self._slots: Dict[tuple, int] = {}
        self._lock = threading.Lock()

    # ---- metadata ----
    def cc_store(self) -> int:
        return 0  # no native Store* behind this tier

    def lookup(self, block_ids: List[bytes]) -> List[bool]:
        with self._lock:
            present = {k[0] for k in self._slots}
        return [bytes(b) in present for b in block_ids]

    def lookup_on_prefix(self, block_ids: List[bytes]) -> int:
        found = -1
        for i, hit in enumerate(self.lookup(block_ids)):
            if not hit:
                break
            found = i
        return found

    def prefetch(self, block_ids: List[bytes]) -> None:
        pass  # single tier: everything present is already in host memory

    # ---- transfers ----
    def _stream(self):
        s = self.streams[self._rr % len(self.streams)]
        self._rr += 1
        return s

    def _addr_rows(self, addrs, n):
        a = np.ascontiguousarray(np.asarray(addrs, dtype=np.uint64)).reshape(n, -1)
        if a.shape[1] != self.sizes.shape[0]:
            raise ValueError(f"expected {self.sizes.shape[0]} pointers per block, got {a.shape[1]}")
        return a

    def _finish(self, stream, task):
        def cb(ok):
            task.ok = bool(ok)
            task.done.set()

        stream.AppendCallback(cb)
        return task

    def dump_data(self, block_ids, shard_index, src_addr, prerequisite_handle: int = 0) -> Task:
        n = len(block_ids)
        rows = self._addr_rows(src_addr, n)
        stream = self._stream()
        stream.WaitEvent(prerequisite_handle)  # Stream::WaitEvent before the first copy
        with self._lock:
            slots = []
            for b, s in zip(block_ids, shard_index):
                key = (bytes(b), int(s))
                if key not in self._slots:
                    if len(self._slots) >= self.capacity:
                        raise RuntimeError("-50009, host store is full")
                    self._slots[key] = len(self._slots)
                slots.append(self._slots[key])
        for row, slot in zip(rows, slots):
            dst = self.slab + slot * self.slot_bytes
            if self.uniform:
                stream.DeviceToHostGatherAsync(row, dst, int(self.sizes[0]), row.shape[0])
            else:
                off = 0
                for p, sz in zip(row, self.sizes):
                    stream.DeviceToHostAsync(int(p), dst + off, int(sz))
                    off += int(sz)
        return self._finish(stream, _Task())

    def load_data(self, block_ids, shard_index, dst_addr) -> Task:
        n = len(block_ids)
        rows = self._addr_rows(dst_addr, n)
        stream = self._stream()
        with self._lock:
            try:
                slots = [self._slots[(bytes(b), int(s))] for b, s in zip(block_ids, shard_index)]
            except KeyError as e:
                raise RuntimeError(f"-50005, block not found: {e}") from None
        for row, slot in zip(rows, slots):
            src = self.slab + slot * self.slot_bytes
            if self.uniform:
                stream.HostToDeviceScatterAsync(src, row, int(self.sizes[0]), row.shape[0])
            else:
                off = 0
                for p, sz in zip(row, self.sizes):
                    stream.HostToDeviceAsync(src + off, int(p), int(sz))
                    off += int(sz)
        return self._finish(stream, _Task())

    def dump(self, block_ids, shard_index, src_tensor) -> Task:
        return self.dump_data(block_ids, shard_index,
                              [[t.data_ptr() for t in row] for row in src_tensor])

    def load(self, block_ids, shard_index, dst_tensor) -> Task:
        return self.load_data(block_ids, shard_index,
                              [[t.data_ptr() for t in row] for row in dst_tensor])

    def wait(self, task: Task) -> None:
        if not task.done.wait(timeout=float(self.config.get("timeout_ms", 30000)) / 1e3):
            raise RuntimeError("-50010, transfer timed out")
        if not task.ok:
            raise RuntimeError("-1, transfer failed")

    def check(self, task: Task) -> bool:
        return task.done.is_set()

    def slot_view(self, block_id: bytes, shard: int = 0):
        """numpy view of a stored slot (for tests and debugging)."""
        slot = self._slots[(bytes(block_id), int(shard))]
        return host_view(self.slab + slot * self.slot_bytes, self.slot_bytes)
