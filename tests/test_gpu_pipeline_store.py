"""GPU tests of the "Cache|Posix" pipeline: paged KV in HBM -> pinned staging (gather kernel) ->
block files in the reference's on-disk format, and back.  The contract is the reference's e2e
test of the same pipeline (ucm/store/test/e2e/cache_on_posix_test.py:45-118): 0 % lookups, dump,
100 % lookups from the worker and from a lookup-only scheduler instance, load, bit-exact
compare."""
import os
import time

import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import posix_format as fmt
from ucm_amd.store import UcmPipelineStore

pytestmark = pytest.mark.gpu

TENSOR, LAYERS = 32768, 8  # a shard = a block = 8 layers x {K, V} x 32 KiB = 512 KiB
SHARD = TENSOR * LAYERS * 2


def config(root, **kw):
    cfg = {"store_pipeline": "Cache|Posix", "storage_backends": [str(root)], "timeout_ms": 10000,
           "tensor_size": TENSOR, "shard_size": SHARD, "block_size": SHARD, "io_direct": False,
           "posix_data_trans_concurrency": 8, "posix_lookup_concurrency": 8, "data_dir_shard_bytes": 2,
           "buffer_capacity_bytes": 64 * SHARD}
    cfg.update(kw)
    return cfg


def rows(n, seed):
    rng = rng_for(seed)
    return [[torch.from_numpy(rng.integers(0, 256, TENSOR, dtype=np.uint8)).cuda() for _ in range(LAYERS * 2)]
            for _ in range(n)]


def block_ids(n, seed):
    rng = rng_for(seed)
    return [bytes(rng.integers(0, 256, 16, dtype=np.uint8)) for _ in range(n)]


def wait_until(pred, seconds=10.0):
    end = time.time() + seconds
    while time.time() < end:
        if pred():
            return True
        time.sleep(0.01)
    return pred()


def test_e2e_like_the_reference(tmp_path):
    worker = UcmPipelineStore(config(tmp_path, device_id=0))
    scheduler = UcmPipelineStore(config(tmp_path))
    n = 32
    ids = block_ids(n, 1)
    assert not any(scheduler.lookup(ids)) and scheduler.lookup_on_prefix(ids) == -1
    assert not any(worker.lookup(ids))
    src = rows(n, 2)
    worker.wait(worker.dump(ids, [0] * n, src))
    assert all(worker.lookup(ids))  # staged shards count as present at once
    # the files appear behind the worker's back; the scheduler sees them once they are renamed
    assert wait_until(lambda: scheduler.lookup_on_prefix(ids) + 1 == n)
    assert all(scheduler.lookup(ids))
    dst = [[torch.zeros_like(t) for t in row] for row in src]
    worker.wait(worker.load(ids, [0] * n, dst))
    torch.cuda.synchronize()
    for ra, rb in zip(src, dst):
        for a, b in zip(ra, rb):
            assert torch.equal(a, b)
    # every file is the block's tensors back to back, as the format says
    for i, row in zip(ids, src):
        got = fmt.read_shard([str(tmp_path)], i, 0, SHARD, TENSOR, 2)
        assert got == [t.cpu().numpy().tobytes() for t in row]
    worker.close()
    scheduler.close()


def test_blocks_come_back_from_files_after_eviction_and_restart(tmp_path):
    # staging holds 8 shards; 24 blocks pass through it, so most loads must read the files
    small = config(tmp_path, device_id=0, buffer_capacity_bytes=8 * SHARD)
    worker = UcmPipelineStore(small)
    n = 24
    ids, src = block_ids(n, 3), rows(n, 4)
    for s in range(0, n, 4):  # four shards per task: what the staging buffer can hold at once
        worker.wait(worker.dump(ids[s:s + 4], [0] * 4, src[s:s + 4]))
        assert wait_until(lambda: all(os.path.exists(fmt.data_file_path([str(tmp_path)], i, False, 2))
                                      for i in ids[s:s + 4]))
    dst = [[torch.zeros_like(t) for t in row] for row in src]
    for s in range(0, n, 4):
        worker.wait(worker.load(ids[s:s + 4], [0] * 4, dst[s:s + 4]))
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for ra, rb in zip(src, dst) for a, b in zip(ra, rb))
    worker.close()
    # a new instance over the same directory (a restarted engine) finds and loads everything
    again = UcmPipelineStore(small)
    assert all(again.lookup(ids))
    dst2 = [[torch.zeros_like(t) for t in row] for row in src[:4]]
    again.wait(again.load(ids[:4], [0] * 4, dst2))
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for ra, rb in zip(src[:4], dst2) for a, b in zip(ra, rb))
    again.close()


def test_loads_blocks_written_in_the_reference_format(tmp_path):
    # files laid down by the format checker (standing for another UCM deployment) reach HBM
    rng = rng_for(5)
    ids = block_ids(6, 6)
    data = {i: {0: [rng.integers(0, 256, TENSOR, dtype=np.uint8).tobytes() for _ in range(LAYERS * 2)]} for i in ids}
    worker = UcmPipelineStore(config(tmp_path, device_id=0))  # creates the shard directories
    for i in ids:
        fmt.write_block([str(tmp_path)], i, data[i], SHARD, 2)
    assert worker.lookup_on_prefix(ids) == 5
    dst = [[torch.zeros(TENSOR, dtype=torch.uint8, device="cuda") for _ in range(LAYERS * 2)] for _ in ids]
    worker.wait(worker.load(ids, [0] * 6, dst))
    torch.cuda.synchronize()
    for i, row in zip(ids, dst):
        assert [t.cpu().numpy().tobytes() for t in row] == data[i][0]
    # a block that is in neither tier fails the load
    missing = block_ids(1, 7)
    with pytest.raises(RuntimeError):
        worker.wait(worker.load(missing, [0], dst[:1]))
    worker.close()


def test_posix_alone_rejects_device_tensors(tmp_path):
    s = UcmPipelineStore(config(tmp_path, store_pipeline="Posix", device_id=0, tensor_size=SHARD))
    with pytest.raises(ValueError, match="host memory"):
        s.dump(block_ids(1, 8), [0], [[torch.zeros(SHARD, dtype=torch.uint8, device="cuda")]])
    t = torch.from_numpy(rng_for(9).integers(0, 256, SHARD, dtype=np.uint8))
    ids = block_ids(1, 10)
    s.wait(s.dump(ids, [0], [[t]]))
    back = torch.zeros_like(t)
    s.wait(s.load(ids, [0], [[back]]))
    assert torch.equal(t, back)
    s.close()
    with pytest.raises(ValueError):
        UcmPipelineStore(config(tmp_path, store_pipeline="Cache|Nfs"))
