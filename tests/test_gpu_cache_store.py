"""GPU tests of the native cache store (csrc/cache_store.hip) through its C ABI.

The contract tested is the one of the reference's CacheStore: the e2e dump -> lookup -> load
round trip (ucm/store/test/e2e/cache_on_empty_test.py:46-79), the staging-buffer semantics of
trans_buffer.cc (dedup of resident shards, ring replacement of unreferenced nodes), the backend
hand-off of dump_queue.cc / load_queue.cc and the task rules of task_wrapper.h.
"""
import threading

import numpy as np
import pytest
import torch

from helpers import rng_for

pytestmark = pytest.mark.gpu

L, NB, CHUNK = 4, 32, 16384  # 4 layers x {K,V}: a shard is 8 pieces of 16 KiB


def make_kv(seed):
    rng = rng_for(seed)
    return [torch.from_numpy(rng.integers(0, 256, size=(2, NB, CHUNK), dtype=np.uint8)).cuda()
            for _ in range(L)]


def addrs(tensors, blocks):
    return np.array([[t[kv, b].data_ptr() for t in tensors for kv in (0, 1)] for b in blocks], np.uint64)


def ids_of(tag, n):
    return [bytes([tag, i]) * 8 for i in range(n)]


def shard_bytes(tensors, block):
    return np.concatenate([t[kv, block].cpu().numpy() for t in tensors for kv in (0, 1)])


class DictBackend:
    """The slower tier: keeps shard bytes in a dict (stands where the reference chains a
    posix store behind the cache store)."""

    def __init__(self):
        self.data = {}
        self.dumps = 0
        self.loads = 0
        self.lock = threading.Lock()

    def lookup(self, ids):
        with self.lock:
            return [(i, 0) in self.data for i in ids]

    def dump(self, ids, shard_idx, views):
        with self.lock:
            for i, s, v in zip(ids, shard_idx, views):
                self.data[(i, s)] = v.copy()
                self.dumps += 1

    def load(self, ids, shard_idx, views):
        with self.lock:
            for i, s, v in zip(ids, shard_idx, views):
                v[:] = self.data[(i, s)]  # KeyError -> the hook reports failure
                self.loads += 1


def make_store(nodes, backend=None, **kw):
    from ucm_amd.store import CacheStore

    cfg = {"tensor_size_list": [CHUNK] * (2 * L), "buffer_capacity_bytes": nodes * 2 * L * CHUNK,
           "timeout_ms": 20000}
    if backend is not None:
        cfg["store_backend"] = backend
    cfg.update(kw)
    return CacheStore(cfg)


def test_dump_lookup_load_roundtrip():
    src, dst = make_kv(1), [torch.zeros((2, NB, CHUNK), dtype=torch.uint8, device="cuda") for _ in range(L)]
    store = make_store(16)
    assert store.nodes == 16
    ids = ids_of(1, 10)
    blocks = [3, 7, 0, 15, 9, 31, 20, 21, 22, 1]
    new_blocks = [2, 4, 5, 6, 8, 10, 11, 12, 13, 14]
    task = store.dump_data(ids, [0] * 10, addrs(src, blocks))
    store.wait(task)
    assert store.lookup(ids + [b"x" * 16]) == [True] * 10 + [False]
    assert store.lookup_on_prefix(ids[:3] + [b"y" * 16] + ids[3:]) == 2
    assert store.lookup_on_prefix([b"y" * 16] + ids) == -1
    task = store.load_data(ids, [0] * 10, addrs(dst, new_blocks))
    assert isinstance(store.check(task), bool)
    store.wait(task)
    for l in range(L):
        assert torch.equal(dst[l][:, new_blocks], src[l][:, blocks])
        rest = [b for b in range(NB) if b not in new_blocks]
        assert not dst[l][:, rest].any()
    # tensor-row form of the interface (ucmstore_v1.py load / dump)
    rows = [[t[kv, b] for t in src for kv in (0, 1)] for b in (23, 24)]
    store.wait(store.dump(ids_of(2, 2), [0, 0], rows))
    out_rows = [[t[kv, b] for t in dst for kv in (0, 1)] for b in (30, 29)]
    store.wait(store.load(ids_of(2, 2), [0, 0], out_rows))
    for l in range(L):
        assert torch.equal(dst[l][:, [30, 29]], src[l][:, [23, 24]])
    store.close()


def test_resident_shard_is_not_copied_again():
    """trans_buffer.cc:480-486 + dump_queue.cc:116-126: a shard that is already staged keeps
    its bytes; only the backend sees the second dump."""
    src = make_kv(2)
    be = DictBackend()
    store = make_store(8, be)
    ids = ids_of(3, 2)
    store.wait(store.dump_data(ids, [0, 0], addrs(src, [5, 6])))
    first = shard_bytes(src, 5)
    src[0][0, 5].fill_(0xEE)  # change the device copy, dump the same block id again
    torch.cuda.synchronize()
    store.wait(store.dump_data(ids, [0, 0], addrs(src, [5, 6])))
    dst = [torch.zeros_like(t) for t in src]
    store.wait(store.load_data(ids[:1], [0], addrs(dst, [0])))
    assert np.array_equal(shard_bytes(dst, 0), first)
    assert be.dumps == 4 and be.loads == 0
    store.close()


def test_ring_replacement_without_a_backend_loses_old_blocks():
    src = make_kv(3)
    store = make_store(8)
    ids = ids_of(4, 12)
    for i in range(12):  # one task each, so that earlier nodes are unreferenced when reused
        store.wait(store.dump_data(ids[i:i + 1], [0], addrs(src, [i])))
    hits = store.lookup(ids)
    assert hits == [False] * 4 + [True] * 8
    dst = [torch.zeros_like(t) for t in src]
    store.wait(store.load_data(ids[4:], [0] * 8, addrs(dst, list(range(8)))))
    for l in range(L):
        assert torch.equal(dst[l][:, :8], src[l][:, 4:12])
    task = store.load_data(ids[:1], [0], addrs(dst, [20]))
    with pytest.raises(RuntimeError):
        store.wait(task)  # in neither tier
    assert not store.lookup(ids[:1])[0]  # the failed load left no stale entry behind
    store.close()


def test_backend_serves_what_the_staging_cache_dropped():
    src = make_kv(4)
    be = DictBackend()
    store = make_store(8, be)
    ids = ids_of(5, 12)
    for i in range(12):
        store.wait(store.dump_data(ids[i:i + 1], [0], addrs(src, [i])))
    assert store.lookup(ids) == [True] * 12  # 4 of them only in the backend
    assert be.dumps == 12
    dst = [torch.zeros_like(t) for t in src]
    store.wait(store.load_data(ids[:4], [0] * 4, addrs(dst, [24, 25, 26, 27])))
    assert be.loads == 4
    for l in range(L):
        assert torch.equal(dst[l][:, 24:28], src[l][:, 0:4])
    # what the backend holds is byte-identical to the device shard
    assert np.array_equal(be.data[(ids[9], 0)], shard_bytes(src, 9))
    # a block the backend does not know fails the task
    with pytest.raises(RuntimeError):
        store.wait(store.load_data([b"q" * 16], [0], addrs(dst, [1])))
    store.close()


def test_dump_waits_for_the_producers_event():
    """dump_queue.cc:101-107: the D2H copy is ordered after the prerequisite event."""
    store = make_store(8)
    kv = [torch.zeros((2, NB, CHUNK), dtype=torch.uint8, device="cuda") for _ in range(L)]
    big = torch.empty(1 << 28, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    ev = torch.cuda.Event()
    with torch.cuda.stream(side):
        for _ in range(8):
            big.add_(1)  # keeps the producer stream busy for a while
        for t in kv:
            t.fill_(0x5A)
        ev.record(side)
    task = store.dump_data(ids_of(6, 1), [0], addrs(kv, [2]), ev.cuda_event)
    store.wait(task)
    dst = [torch.zeros_like(t) for t in kv]
    store.wait(store.load_data(ids_of(6, 1), [0], addrs(dst, [0])))
    assert (shard_bytes(dst, 0) == 0x5A).all()
    store.close()


def test_shards_of_one_block_and_mixed_tensor_sizes():
    from ucm_amd.store import CacheStore

    sizes = [4096, 12288, 4096, 1000]  # two launches: 4096-byte pieces and the others
    store = CacheStore({"tensor_size_list": sizes, "buffer_capacity_bytes": 64 * sum(sizes)})
    rng = rng_for(5)
    n = 6
    src = [torch.from_numpy(rng.integers(0, 256, size=(n, s), dtype=np.uint8)).cuda() for s in sizes]
    dst = [torch.zeros_like(t) for t in src]
    block = b"B" * 16
    a = np.array([[t[i].data_ptr() for t in src] for i in range(n)], np.uint64)
    b = np.array([[t[n - 1 - i].data_ptr() for t in dst] for i in range(n)], np.uint64)
    store.wait(store.dump_data([block] * n, list(range(n)), a))  # six shards of one block
    assert store.lookup([block]) == [True]
    store.wait(store.load_data([block] * n, list(range(n)), b))
    for t_src, t_dst in zip(src, dst):
        assert torch.equal(t_dst, torch.flip(t_src, dims=[0]))
    store.close()


def test_task_rules_and_argument_errors():
    store = make_store(8)
    from ucm_amd.store.cache_store import CacheTask

    with pytest.raises(RuntimeError):
        store.wait(CacheTask(12345))          # unknown id (task_wrapper.h:79)
    with pytest.raises(RuntimeError):
        store.check(CacheTask(12345))
    src = make_kv(6)
    t = store.dump_data(ids_of(7, 1), [0], addrs(src, [0]))
    store.wait(t)
    with pytest.raises(RuntimeError):
        store.wait(t)                          # Wait forgets the task
    with pytest.raises(ValueError):
        store.dump_data(ids_of(7, 1), [0], np.zeros((1, 3), np.uint64))
    with pytest.raises(ValueError):
        store.dump_data([b"short"], [0], addrs(src, [0]))
    with pytest.raises(ValueError):
        store.dump_data(ids_of(7, 2), [0], addrs(src, [0, 1]))
    with pytest.raises(ValueError):
        bad = addrs(src, [0])
        bad[0, 3] = 0
        store.dump_data(ids_of(7, 1), [0], bad)   # null device address
    store.wait(store.dump_data([], [], np.zeros((0, 2 * L), np.uint64)))  # empty task
    store.close()
    from ucm_amd.store import CacheStore

    with pytest.raises(ValueError):
        CacheStore({"tensor_size_list": [], "buffer_capacity_bytes": 1 << 20})
    with pytest.raises(ValueError):
        CacheStore({"tensor_size_list": [1 << 20], "buffer_capacity_bytes": 1 << 10})
    with pytest.raises(ValueError):
        CacheStore({"tensor_size": 3, "shard_size": 10, "buffer_capacity_bytes": 1 << 20})


def test_many_tasks_in_flight_from_two_threads():
    """Dumps and loads submitted concurrently: every load of a dumped block returns its bytes."""
    src = make_kv(7)
    store = make_store(64)
    ids = ids_of(8, NB)
    store.wait(store.dump_data(ids[:16], [0] * 16, addrs(src, list(range(16)))))
    dst = [torch.zeros_like(t) for t in src]
    errors = []

    def dumper():
        try:
            tasks = [store.dump_data(ids[i:i + 1], [0], addrs(src, [i])) for i in range(16, NB)]
            for t in tasks:
                store.wait(t)
        except Exception as e:  # pragma: no cover
            errors.append(e)

    def loader():
        try:
            tasks = [store.load_data(ids[i:i + 1], [0], addrs(dst, [i])) for i in range(16)]
            for t in tasks:
                store.wait(t)
        except Exception as e:  # pragma: no cover
            errors.append(e)

    th = [threading.Thread(target=dumper), threading.Thread(target=loader)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not errors
    for l in range(L):
        assert torch.equal(dst[l][:, :16], src[l][:, :16])
    assert store.lookup(ids) == [True] * NB
    store.close()
