"""Device <-> host KV block transfer ("trans") with the method names of the reference's
`ucmtrans` binding (ucm/shared/trans/cpy/trans.py.cc:164-192): Device.Setup / MakeStream /
MakeSMStream and the twelve Stream copy methods plus Synchronized.

Pointers are plain integers.  A pointer table is either a numpy uint64 array (host table) or
an integer address of a table that already lives in device-readable memory
(trans.py.cc:40-160 makes the same distinction).  Failures raise RuntimeError / ValueError.
"""
import ctypes as C

import numpy as np

from . import _lib


def _table(obj):
    """-> (address, on_device, keepalive)"""
    if isinstance(obj, np.ndarray):
        if obj.dtype != np.uint64:
            raise ValueError("pointer tables must be numpy uint64 arrays")
        arr = np.ascontiguousarray(obj)
        return arr.ctypes.data, 0, arr
    return int(obj), 1, None


class Stream:
    def __init__(self, kind):
        h = C.c_void_p()
        _lib.check(_lib.lib().ucm_trans_stream_create(kind, C.byref(h)))
        self._h = h
        self.kind = kind
        self._callbacks = []

    def close(self):
        if self._h is not None and _lib._lib is not None:
            _lib.lib().ucm_trans_stream_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self):
        """The hipStream_t as an integer."""
        return _lib.lib().ucm_trans_stream_handle(self._h)

    # ---- single copies ----
    def DeviceToHost(self, src, dst, size):
        _lib.check(_lib.lib().ucm_trans_d2h(self._h, src, dst, size, 1))

    def DeviceToHostAsync(self, src, dst, size):
        _lib.check(_lib.lib().ucm_trans_d2h(self._h, src, dst, size, 0))

    def HostToDevice(self, src, dst, size):
        _lib.check(_lib.lib().ucm_trans_h2d(self._h, src, dst, size, 1))

    def HostToDeviceAsync(self, src, dst, size):
        _lib.check(_lib.lib().ucm_trans_h2d(self._h, src, dst, size, 0))

    # ---- pointer-table copies ----
    def _batch(self, src, dst, size, number, sync):
        sa, son, k1 = _table(src)
        da, don, k2 = _table(dst)
        if son != don:
            raise ValueError("source and destination tables must both be host or both be device")
        _lib.check(_lib.lib().ucm_trans_batch(self._h, sa, da, son, size, number, sync))

    def _gather(self, src, dst, size, number, sync):
        sa, son, k1 = _table(src)
        _lib.check(_lib.lib().ucm_trans_gather(self._h, sa, son, int(dst), size, number, sync))

    def _scatter(self, src, dst, size, number, sync):
        da, don, k2 = _table(dst)
        _lib.check(_lib.lib().ucm_trans_scatter(self._h, int(src), da, don, size, number, sync))

    def DeviceToHostBatch(self, src, dst, size, number):
        self._batch(src, dst, size, number, 1)

    def DeviceToHostBatchAsync(self, src, dst, size, number):
        self._batch(src, dst, size, number, 0)

    def DeviceToHostGather(self, src, dst, size, number):
        self._gather(src, dst, size, number, 1)

    def DeviceToHostGatherAsync(self, src, dst, size, number):
        self._gather(src, dst, size, number, 0)

    def HostToDeviceBatch(self, src, dst, size, number):
        self._batch(src, dst, size, number, 1)

    def HostToDeviceBatchAsync(self, src, dst, size, number):
        self._batch(src, dst, size, number, 0)

    def HostToDeviceScatter(self, src, dst, size, number):
        self._scatter(src, dst, size, number, 1)

    def HostToDeviceScatterAsync(self, src, dst, size, number):
        self._scatter(src, dst, size, number, 0)

    # ---- table-free paged form (address rule of KVCacheLayout.extract_block_addrs,
    #      ucm/integration/vllm/ucm_connector.py:135-148) ----
    def PagedGatherAsync(self, base_ptrs, col_bytes, block_ids, dst, sync=False, num_cache_blocks=0):
        self._paged(base_ptrs, col_bytes, block_ids, dst, 0, sync, num_cache_blocks)

    def PagedScatterAsync(self, src, base_ptrs, col_bytes, block_ids, sync=False, num_cache_blocks=0):
        self._paged(base_ptrs, col_bytes, block_ids, src, 1, sync, num_cache_blocks)

    def _paged(self, base_ptrs, col_bytes, block_ids, flat, to_cache, sync, num_cache_blocks=0):
        """num_cache_blocks: blocks every column holds; ids outside [0, num_cache_blocks) are
        refused (0 = unknown: only negative ids are)."""
        base = np.ascontiguousarray(base_ptrs, dtype=np.uint64).reshape(-1)
        cb = np.ascontiguousarray(col_bytes, dtype=np.uint64).reshape(-1)
        ids = np.ascontiguousarray(block_ids, dtype=np.int32).reshape(-1)
        if base.shape != cb.shape:
            raise ValueError("base_ptrs and col_bytes must have the same length")
        _lib.check(_lib.lib().ucm_trans_paged_copy(self._h, base.ctypes.data, cb.ctypes.data,
                                                   base.shape[0], ids.ctypes.data, ids.shape[0],
                                                   int(num_cache_blocks), int(flat), to_cache,
                                                   int(bool(sync))))

    # ---- ordering ----
    def Synchronized(self):
        _lib.check(_lib.lib().ucm_trans_stream_sync(self._h))

    def WaitEvent(self, event):
        """event: a hipEvent_t as an integer (torch.cuda.Event.cuda_event), 0/None = no-op
        (Stream::WaitEvent, ucm/shared/trans/cuda/cuda_stream.cc:158-164)."""
        _lib.check(_lib.lib().ucm_trans_stream_wait_event(self._h, event or None))

    def AppendCallback(self, fn):
        """fn(ok: bool) runs on a runtime thread after all enqueued work
        (Stream::AppendCallback, cuda_stream.cc:139-149)."""
        proto = C.CFUNCTYPE(None, C.c_int, C.c_void_p)

        def tramp(ok, _user):
            fn(bool(ok))

        cb = proto(tramp)
        self._callbacks.append(cb)  # keep the thunk alive
        _lib.check(_lib.lib().ucm_trans_stream_append_callback(self._h, C.cast(cb, C.c_void_p), None))


class Buffer:
    """Pinned host / device allocations (UC::Trans::Buffer, ucm/shared/trans/buffer.h:32-47)."""

    def __init__(self):
        self._host, self._dev = [], []

    def MakeHostBuffer(self, size):
        p = C.c_void_p()
        _lib.check(_lib.lib().ucm_trans_host_alloc(size, C.byref(p)))
        self._host.append(p.value)
        return p.value

    def MakeDeviceBuffer(self, size):
        p = C.c_void_p()
        _lib.check(_lib.lib().ucm_trans_device_alloc(size, C.byref(p)))
        self._dev.append(p.value)
        return p.value

    def release(self):
        for p in self._host:
            _lib.lib().ucm_trans_host_free(p)
        for p in self._dev:
            _lib.lib().ucm_trans_device_free(p)
        self._host, self._dev = [], []

    def __del__(self):
        try:
            if _lib._lib is not None:
                self.release()
        except Exception:
            pass


class Device:
    def Setup(self, device_id):
        _lib.check(_lib.lib().ucm_trans_setup(int(device_id)))

    def MakeStream(self):
        return Stream(_lib.TRANS_CE)

    def MakeSMStream(self):
        return Stream(_lib.TRANS_SM)

    def MakeBuffer(self):
        return Buffer()


def host_view(ptr, nbytes):
    """numpy uint8 view of `nbytes` of host memory at integer address `ptr`."""
    return np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(ptr))
