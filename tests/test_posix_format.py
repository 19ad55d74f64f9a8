"""CPU tests: the posix on-disk format checker (oracle/posix_format.py) against the expectations
the reference's own tests state, and the native store (host-only part of the C-ABI library)
against the checker, file by file and byte by byte."""
import os
import time

import numpy as np
import pytest

from oracle import posix_format as fmt
from ucm_amd.store import PosixStore

BLOCK = bytes.fromhex("a1b2c3d4e5f6789012345678901234ab")  # the id the reference's tests use


def rnd_id(rng):
    return bytes(rng.integers(0, 256, 16, dtype=np.uint8))


def store(tmp_path, **kw):
    cfg = {"storage_backends": [str(tmp_path)], "device_id": 0, "tensor_size": 4096, "shard_size": 4096,
           "block_size": 4096, "data_dir_shard_bytes": 0, "posix_data_trans_concurrency": 4,
           "posix_lookup_concurrency": 4}
    cfg.update(kw)
    return PosixStore(cfg)


def host(n, seed):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


# ---- the checker against the reference's stated expectations ----
def test_checker_paths_match_the_reference_tests():
    # posix_space_manager_test.cc:73-84: "{}data/{:02x}.tmp" and "{}data/{:02x}" of the id bytes
    root = "/some/backend/"
    hexname = "a1b2c3d4e5f6789012345678901234ab"
    assert fmt.file_name(BLOCK) == hexname
    assert fmt.data_file_path([root], BLOCK, True, 0) == root + "data/" + hexname + ".tmp"
    assert fmt.data_file_path([root], BLOCK, False, 0) == root + "data/" + hexname
    # :96-110: with dataDirShardBytes = 2 the directory is the first two digits of the name
    assert fmt.data_file_path([root], BLOCK, True, 2) == root + "a1/" + hexname + ".tmp"
    assert fmt.data_file_path([root], BLOCK, False, 2) == root + "a1/" + hexname
    # a backend path without the trailing slash gets one (space_layout.cc:121-122)
    assert fmt.data_file_path(["/x"], BLOCK, False, 3) == "/x/a1b/" + hexname
    # leading zeros are kept: two digits per byte
    assert fmt.file_name(bytes(range(16))) == "000102030405060708090a0b0c0d0e0f"


# ---- the native store against the checker ----
@pytest.mark.parametrize("digits", [0, 1, 2, 3])
def test_data_file_path(tmp_path, digits):
    s = store(tmp_path, data_dir_shard_bytes=digits)
    rng = np.random.default_rng(digits)
    for bid in [BLOCK, bytes(16), bytes([255] * 16)] + [rnd_id(rng) for _ in range(20)]:
        for activated in (False, True):
            assert s.data_file_path(bid, activated) == fmt.data_file_path([str(tmp_path)], bid, activated, digits)
    # the first backend gets its shard directories at setup (space_layout.cc:137-147)
    want = {"data"} if digits == 0 else {f"{i:0{digits}x}" for i in range(16 ** digits)}
    assert set(os.listdir(tmp_path)) == want
    s.close()


def test_several_backends_choose_by_the_standard_hash(tmp_path):
    roots = [tmp_path / f"b{i}" for i in range(3)]
    for r in roots:
        (r / "data").mkdir(parents=True)  # secondary backends must already hold the directories
    s = store(tmp_path, storage_backends=[str(r) for r in roots])
    rng = np.random.default_rng(1)
    used = set()
    for _ in range(64):
        bid = rnd_id(rng)
        p = s.data_file_path(bid)
        assert p == fmt.data_file_path([str(r) for r in roots], bid, False, 0)
        used.add(p.split("/data/")[0])
    assert len(used) == 3
    s.close()
    # a secondary backend without the directories is refused (space_layout.cc:150-162)
    (tmp_path / "empty").mkdir()
    with pytest.raises(RuntimeError):
        store(tmp_path, storage_backends=[str(roots[0]), str(tmp_path / "empty")])


def test_setup_with_invalid_param(tmp_path):
    # posix_store_test.cc:34-62
    with pytest.raises(ValueError):
        PosixStore({})
    with pytest.raises(ValueError):
        PosixStore({"storage_backends": [str(tmp_path)], "device_id": 0})  # sizes missing
    with pytest.raises(ValueError):
        store(tmp_path, posix_data_trans_concurrency=0)
    with pytest.raises(ValueError):
        store(tmp_path, posix_lookup_concurrency=0)
    with pytest.raises(ValueError):
        store(tmp_path, data_dir_shard_bytes=6)
    with pytest.raises(ValueError):
        store(tmp_path, tensor_size=4096, shard_size=6000)  # not a multiple
    with pytest.raises(ValueError):
        store(tmp_path, posix_io_engine="uring")
    with pytest.raises(RuntimeError):
        store(tmp_path, storage_backends=[str(tmp_path / "missing")])  # mkdir of its shard dir fails


def test_commit_makes_a_file_visible(tmp_path):
    # posix_space_manager_test.cc:64-88
    s = store(tmp_path)
    activated = s.data_file_path(BLOCK, True)
    assert not os.path.exists(activated)
    open(activated, "wb").close()
    assert s.lookup([BLOCK]) == [False]
    s.commit(BLOCK, True)
    assert s.lookup([BLOCK]) == [True]
    assert not os.path.exists(activated) and os.path.exists(s.data_file_path(BLOCK, False))
    # a failed commit removes the .tmp file; committing nothing reports the missing file
    other = bytes(range(16))
    open(s.data_file_path(other, True), "wb").close()
    s.commit(other, False)
    assert not os.path.exists(s.data_file_path(other, True)) and s.lookup([other]) == [False]
    with pytest.raises(RuntimeError):
        s.commit(other, True)
    s.close()


def test_lookup_reports_the_leading_run(tmp_path):
    # posix_space_manager_test.cc:113-160
    s = store(tmp_path)
    rng = np.random.default_rng(2)
    blocks = [rnd_id(rng) for _ in range(3)]
    assert s.lookup_on_prefix(blocks) == -1 and s.lookup(blocks) == [False] * 3
    for b in blocks:
        open(s.data_file_path(b), "wb").close()
    assert s.lookup_on_prefix(blocks) == 2 and s.lookup(blocks) == [True] * 3
    blocks.insert(2, rnd_id(rng))
    assert s.lookup_on_prefix(blocks) == 1
    assert s.lookup(blocks) == [True, True, False, False]  # present blocks after a miss count as absent
    assert s.lookup_on_prefix([]) == -1 and s.lookup([]) == []
    many = [rnd_id(rng) for _ in range(200)]
    for b in many[:150]:
        open(s.data_file_path(b), "wb").close()
    assert s.lookup_on_prefix(many) == 149
    s.close()


def test_dump_then_load(tmp_path):
    # posix_store_test.cc:63-102, and the file is what the checker says it is
    size = 32768
    s = store(tmp_path, tensor_size=size, shard_size=size, block_size=size)
    assert s.lookup([BLOCK]) == [False]
    src = host(size, 3)
    t = s.dump_data([BLOCK], [0], [[src.ctypes.data]])
    s.wait(t)
    assert s.lookup([BLOCK]) == [True]
    with open(fmt.data_file_path([str(tmp_path)], BLOCK, False, 0), "rb") as f:
        assert f.read() == src.tobytes()
    assert oct(os.stat(s.data_file_path(BLOCK)).st_mode & 0o777) == oct(0o644 & ~_umask())
    dst = np.zeros(size, np.uint8)
    t = s.load_data([BLOCK], [0], [[dst.ctypes.data]])
    assert s.check(t) in (False, True)
    s.wait(t)
    assert np.array_equal(src, dst)
    with pytest.raises(RuntimeError):
        s.wait(t)  # forgotten after the first wait
    s.close()


def _umask():
    m = os.umask(0)
    os.umask(m)
    return m


def test_layerwise_shards_and_tensors(tmp_path):
    # posix_trans_queue_test.cc:71-118 (eight shards of one block, one task), here with two
    # tensors per shard; the rename happens once, after the last shard
    ts, per, n_shards = 4096, 2, 8
    s = store(tmp_path, tensor_size=ts, shard_size=ts * per, block_size=ts * per * n_shards)
    bufs = [[host(ts, 100 + 10 * i + j) for j in range(per)] for i in range(n_shards)]
    t = s.dump_data([BLOCK] * n_shards, list(range(n_shards)), [[b.ctypes.data for b in row] for row in bufs])
    s.wait(t)
    assert not os.path.exists(s.data_file_path(BLOCK, True))
    for i in range(n_shards):
        got = fmt.read_shard([str(tmp_path)], BLOCK, i, ts * per, ts, 0)
        assert got == [b.tobytes() for b in bufs[i]]
    assert os.path.getsize(s.data_file_path(BLOCK)) == ts * per * n_shards
    out = [[np.zeros(ts, np.uint8) for _ in range(per)] for _ in range(n_shards)]
    order = [5, 0, 7, 2, 1, 6, 3, 4]
    t = s.load_data([BLOCK] * n_shards, order, [[b.ctypes.data for b in out[i]] for i in order])
    s.wait(t)
    for i in range(n_shards):
        for j in range(per):
            assert np.array_equal(out[i][j], bufs[i][j])
    s.close()


def test_a_block_is_invisible_until_its_last_shard(tmp_path):
    ts = 4096
    s = store(tmp_path, tensor_size=ts, shard_size=ts, block_size=ts * 2)
    a, b = host(ts, 5), host(ts, 6)
    s.wait(s.dump_data([BLOCK], [0], [[a.ctypes.data]]))
    assert s.lookup([BLOCK]) == [False] and os.path.exists(s.data_file_path(BLOCK, True))
    s.wait(s.dump_data([BLOCK], [1], [[b.ctypes.data]]))
    assert s.lookup([BLOCK]) == [True]
    with open(s.data_file_path(BLOCK), "rb") as f:
        assert f.read() == a.tobytes() + b.tobytes()
    s.close()


def test_reads_files_written_in_the_reference_format(tmp_path):
    # the other direction of interoperability: files laid down by the checker load bit-exactly
    ts, per, n_shards, digits = 4096, 3, 2, 2
    (tmp_path / "x").mkdir()
    s = store(tmp_path / "x", tensor_size=ts, shard_size=ts * per, block_size=ts * per * n_shards,
              data_dir_shard_bytes=digits)
    rng = np.random.default_rng(7)
    blocks = [rnd_id(rng) for _ in range(5)]
    data = {b: {i: [host(ts, hash((b, i, j)) & 0xffff).tobytes() for j in range(per)] for i in range(n_shards)}
            for b in blocks}
    for b in blocks:
        fmt.write_block([str(tmp_path / "x")], b, data[b], ts * per, digits)
    assert s.lookup(blocks) == [True] * 5
    for b in blocks:
        for i in range(n_shards):
            out = [np.zeros(ts, np.uint8) for _ in range(per)]
            s.wait(s.load_data([b], [i], [[o.ctypes.data for o in out]]))
            assert [o.tobytes() for o in out] == data[b][i]
    s.close()


def test_load_of_a_missing_block_fails_the_task(tmp_path):
    s = store(tmp_path)
    dst = np.zeros(4096, np.uint8)
    t = s.load_data([BLOCK], [0], [[dst.ctypes.data]])
    with pytest.raises(RuntimeError):
        s.wait(t)
    with pytest.raises(ValueError):
        s.load_data([BLOCK], [1], [[dst.ctypes.data]])  # shard index outside the block
    with pytest.raises(RuntimeError):
        s.check(type(t)(12345))
    s.close()


def test_lookup_only_side_cannot_transfer_and_touches_files(tmp_path):
    worker = store(tmp_path)
    src = host(4096, 8)
    worker.wait(worker.dump_data([BLOCK], [0], [[src.ctypes.data]]))
    path = worker.data_file_path(BLOCK)
    os.utime(path, (1_000_000, 1_000_000))
    sched = PosixStore({"storage_backends": [str(tmp_path)], "data_dir_shard_bytes": 0})  # device_id -1
    with pytest.raises(RuntimeError, match="transfer is not enable"):
        sched.dump_data([BLOCK], [0], [[src.ctypes.data]])
    assert sched.lookup([BLOCK]) == [True]
    deadline = time.time() + 5
    while os.stat(path).st_mtime == 1_000_000 and time.time() < deadline:
        time.sleep(0.01)
    assert os.stat(path).st_mtime > 1_000_000  # hotness tracker (hotness_tracker.cc:60-82)
    # the worker side does not touch
    os.utime(path, (1_000_000, 1_000_000))
    assert worker.lookup([BLOCK]) == [True]
    time.sleep(0.05)
    assert os.stat(path).st_mtime == 1_000_000
    sched.close()
    worker.close()


def test_io_direct(tmp_path):
    # posix_store_test.cc:103-150; some file systems (tmpfs) refuse O_DIRECT at open
    probe = tmp_path / "probe"
    try:
        fd = os.open(probe, os.O_CREAT | os.O_WRONLY | os.O_DIRECT)
        os.close(fd)
    except OSError:
        pytest.skip("this file system refuses O_DIRECT")
    os.remove(probe)
    size = 32768
    s = store(tmp_path, tensor_size=size, shard_size=size, block_size=size, io_direct=True)
    raw = np.zeros(2 * size + 4096, np.uint8)
    off = (-raw.ctypes.data) % 4096
    a, b = raw[off:off + size], raw[off + size:off + 2 * size]
    a[:] = host(size, 9)
    s.wait(s.dump_data([BLOCK], [0], [[a.ctypes.data]]))
    s.wait(s.load_data([BLOCK], [0], [[b.ctypes.data]]))
    assert np.array_equal(a, b)
    s.close()


def test_garbage_collection_removes_the_oldest_files(tmp_path):
    # 16 directories (one hex digit); capacity 160 blocks -> 10 files per directory, trigger at
    # 0.5 -> 5; recycle 40 % of a directory's files per pass (shard_gc.cc:31-53, 118-149)
    bs = 4096
    s = store(tmp_path, data_dir_shard_bytes=1, capacity_bytes=160 * bs, posix_gc_trigger_threshold_ratio=0.5,
              posix_gc_recycle_percent=0.4, posix_gc_shard_sample_ratio=1.0, posix_gc_check_interval_sec=3600)
    src = host(bs, 10)
    ids = []
    for d in range(16):
        for i in range(6):
            bid = bytes([d << 4 | i]) + bytes(15)
            ids.append(bid)
            s.wait(s.dump_data([bid], [0], [[src.ctypes.data]]))
            os.utime(s.data_file_path(bid), (1_000_000 + i, 1_000_000 + i))  # i = age order
    assert s.gc_once() == 16 * 2  # 6 files >= 5: one pass removes int(6 * 0.4) = 2 per directory, then 4 < 5
    for bid in ids:
        age = bid[0] & 15
        assert os.path.exists(s.data_file_path(bid)) == (age >= 2)  # the two oldest went
    assert s.gc_once() == 0
    s.close()
    plain = store(tmp_path)
    with pytest.raises(NotImplementedError):
        plain.gc_once()
    plain.close()
    with pytest.raises(ValueError):
        store(tmp_path, data_dir_shard_bytes=1, capacity_bytes=16 * bs)  # cannot recycle anything


def test_many_tasks_from_several_threads(tmp_path):
    import threading
    ts = 8192
    s = store(tmp_path, tensor_size=ts, shard_size=ts, block_size=ts, data_dir_shard_bytes=2)
    errors = []

    def work(seed):
        try:
            rng = np.random.default_rng(seed)
            ids = [rnd_id(rng) for _ in range(40)]
            bufs = [host(ts, seed * 1000 + i) for i in range(40)]
            s.wait(s.dump_data(ids, [0] * 40, [[b.ctypes.data] for b in bufs]))
            outs = [np.zeros(ts, np.uint8) for _ in range(40)]
            s.wait(s.load_data(ids, [0] * 40, [[o.ctypes.data] for o in outs]))
            assert all(np.array_equal(a, b) for a, b in zip(bufs, outs))
            assert s.lookup_on_prefix(ids) == 39
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    s.close()
