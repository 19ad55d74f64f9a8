"""GPU parity: KV block gather / scatter through the C ABI, byte-exact against memcpy
semantics (the oracle's pointer-table loops) and the reference's own round-trip pattern
(ucm/shared/test/case/trans/trans_test.cc:29-141)."""
import threading

import numpy as np
import pytest
import torch

from helpers import rng_for
from oracle import c_api

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    from ucm_amd.trans import Device

    d = Device()
    d.Setup(0)
    return d


def pinned(nbytes):
    return torch.empty(nbytes, dtype=torch.uint8).pin_memory()


def ptrs_of(t, ids, stride):
    return np.array([t.data_ptr() + int(i) * stride for i in ids], dtype=np.uint64)


@pytest.mark.parametrize("kind", ["ce", "sm"])
def test_roundtrip_like_the_reference_unit_test(device, kind):
    """64*61 chunks of 36 KiB: scatter host->device, gather device->host, compare everything
    (the reference compares the first word of each chunk)."""
    size, number = 36 * 1024, 64 * 61
    stream = device.MakeStream() if kind == "ce" else device.MakeSMStream()
    h1, h2 = pinned(size * number), pinned(size * number)
    h1v = h1.numpy()
    h1v[:] = rng_for(1).integers(0, 256, size=size * number, dtype=np.uint8)
    h1v.view(np.uint64).reshape(number, -1)[:, 0] = np.arange(number)
    pool = torch.zeros(size * number, dtype=torch.uint8, device="cuda")
    perm = rng_for(2).permutation(number)
    table = ptrs_of(pool, perm, size)
    torch.cuda.synchronize()
    stream.HostToDeviceScatterAsync(h1.data_ptr(), table, size, number)
    stream.DeviceToHostGatherAsync(table, h2.data_ptr(), size, number)
    stream.Synchronized()
    assert np.array_equal(h2.numpy(), h1v)
    # and the device pool holds chunk i at slot perm[i]
    got = pool.cpu().numpy().reshape(number, size)
    assert np.array_equal(got[perm], h1v.reshape(number, size))


def test_sm_stream_with_device_resident_tables_and_batch(device):
    size, number = 4096 + 48, 300  # not a multiple of the 16 KiB segment, 16-byte multiple
    stream = device.MakeSMStream()
    rng = rng_for(3)
    src = torch.from_numpy(rng.integers(0, 256, size=(number + 5) * size, dtype=np.uint8)).cuda()
    dst = torch.zeros((number + 9) * size, dtype=torch.uint8, device="cuda")
    ids_s = rng.permutation(number + 5)[:number]
    ids_d = rng.permutation(number + 9)[:number]
    ts = torch.from_numpy(ptrs_of(src, ids_s, size).view(np.int64)).cuda()
    td = torch.from_numpy(ptrs_of(dst, ids_d, size).view(np.int64)).cuda()
    torch.cuda.synchronize()
    stream.DeviceToHostBatch(ts.data_ptr(), td.data_ptr(), size, number)
    s, d = src.cpu().numpy().reshape(-1, size), dst.cpu().numpy().reshape(-1, size)
    assert np.array_equal(d[ids_d], s[ids_s])
    rest = np.setdiff1d(np.arange(number + 9), ids_d)
    assert not d[rest].any()
    # gather with a device table into a device flat buffer
    flat = torch.zeros(number * size, dtype=torch.uint8, device="cuda")
    stream.DeviceToHostGather(ts.data_ptr(), flat.data_ptr(), size, number)
    assert np.array_equal(flat.cpu().numpy().reshape(number, size), s[ids_s])


@pytest.mark.parametrize("size", [1, 7, 16, 100, 16384, 16385, 70001])
def test_odd_sizes_and_unaligned_chunks(device, size):
    """Any byte count moves completely (the reference's kernel drops a tail < 32 B,
    ucm/shared/trans/cuda/cuda_sm_kernel.cu:56; this one must not)."""
    number = 13
    stream = device.MakeSMStream()
    rng = rng_for(size)
    pool = torch.from_numpy(rng.integers(0, 256, size=(number * (size + 3) + 64), dtype=np.uint8)).cuda()
    table = np.array([pool.data_ptr() + 1 + i * (size + 3) for i in range(number)], np.uint64)
    host = pinned(size * number)
    host.numpy()[:] = 0
    stream.DeviceToHostGather(table, host.data_ptr(), size, number)
    p = pool.cpu().numpy()
    expect = np.concatenate([p[1 + i * (size + 3): 1 + i * (size + 3) + size] for i in range(number)])
    assert np.array_equal(host.numpy(), expect)


def test_kv_cache_gather_scatter_small_config4(device):
    """BASELINE.json config 4 at reduced size: layers x {K,V} x [NB,BS,H,D] bf16 cache; gather the
    selected blocks of several requests into one pinned buffer, scatter into fresh blocks of
    a second cache, compare byte for byte, check untouched blocks stay untouched."""
    L, NB, BS, H, D = 4, 24, 16, 8, 128
    chunk = BS * H * D * 2
    rng = rng_for(4)
    src = [torch.from_numpy(rng.integers(0, 2**16, size=(2, NB, BS, H, D), dtype=np.uint16)
                            .view(np.int16)).cuda() for _ in range(L)]
    dst = [torch.full((2, NB, BS, H, D), 0x5A5A, dtype=torch.int16, device="cuda") for _ in range(L)]
    base_s = np.array([[t[0].data_ptr(), t[1].data_ptr()] for t in src], np.uint64)
    base_d = np.array([[t[0].data_ptr(), t[1].data_ptr()] for t in dst], np.uint64)
    sizes = np.full((L, 2), chunk, np.uint64)
    n_req, n_sel = 3, 5
    old = np.stack([rng.choice(NB, n_sel, replace=False) for _ in range(n_req)]).reshape(-1)
    new = rng.choice(NB, n_req * n_sel, replace=False)
    # address table exactly as KVCacheLayout.extract_block_addrs builds it
    addr_s = c_api.block_addrs(base_s.reshape(-1), sizes.reshape(-1), old)
    addr_d = c_api.block_addrs(base_d.reshape(-1), sizes.reshape(-1), new)
    host = pinned(addr_s.size * chunk)
    stream = device.MakeSMStream()
    torch.cuda.synchronize()
    stream.DeviceToHostGatherAsync(addr_s.reshape(-1), host.data_ptr(), chunk, addr_s.size)
    stream.Synchronized()
    hv = host.numpy().reshape(len(old), L, 2, chunk)
    for i, b in enumerate(old):
        for l in range(L):
            for kv in range(2):
                assert np.array_equal(hv[i, l, kv], src[l][kv, b].cpu().numpy().view(np.uint8).reshape(-1))
    stream.HostToDeviceScatterAsync(host.data_ptr(), addr_d.reshape(-1), chunk, addr_d.size)
    stream.Synchronized()
    for l in range(L):
        d = dst[l].cpu().numpy()
        s = src[l].cpu().numpy()
        assert np.array_equal(d[:, new], s[:, old])
        rest = np.setdiff1d(np.arange(NB), new)
        assert np.all(d[:, rest] == 0x5A5A)
    # the table-free paged form gives the same bytes
    host2 = pinned(addr_s.size * chunk)
    stream.PagedGatherAsync(base_s.reshape(-1), sizes.reshape(-1), old, host2.data_ptr(), sync=True)
    assert np.array_equal(host2.numpy(), host.numpy())
    dst2 = [torch.zeros_like(t) for t in dst]
    base_d2 = np.array([[t[0].data_ptr(), t[1].data_ptr()] for t in dst2], np.uint64)
    stream.PagedScatterAsync(host2.data_ptr(), base_d2.reshape(-1), sizes.reshape(-1), new, sync=True)
    for l in range(L):
        assert np.array_equal(dst2[l].cpu().numpy()[:, new], src[l].cpu().numpy()[:, old])


def test_paged_copy_variable_column_sizes(device):
    """Columns of different sizes (k, v, rope ...): offsets accumulate inside a block row
    (ucm/store/cache/cc/dump_queue.cc:145-161)."""
    rng = rng_for(5)
    col_bytes = [4096, 512, 20000]
    NB = 9
    cols = [torch.from_numpy(rng.integers(0, 256, size=(NB, cb), dtype=np.uint8)).cuda()
            for cb in col_bytes]
    base = [c.data_ptr() for c in cols]
    ids = np.array([7, 0, 3, 3], np.int32)
    host = pinned(len(ids) * sum(col_bytes))
    stream = device.MakeSMStream()
    torch.cuda.synchronize()
    stream.PagedGatherAsync(base, col_bytes, ids, host.data_ptr(), sync=True)
    expect = np.concatenate([np.concatenate([c[i].cpu().numpy() for c in cols]) for i in ids])
    assert np.array_equal(host.numpy(), expect)


def test_wait_event_and_callback(device):
    stream = device.MakeSMStream()
    n = 1 << 20
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    host = pinned(n)
    host.numpy()[:] = 0
    src.fill_(7)  # on torch's current stream
    ev = torch.cuda.Event()
    ev.record()
    stream.WaitEvent(ev.cuda_event)
    done = threading.Event()
    result = []
    stream.DeviceToHostGatherAsync(np.array([src.data_ptr()], np.uint64), host.data_ptr(), n, 1)
    stream.AppendCallback(lambda ok: (result.append(ok), done.set()))
    assert done.wait(30)
    assert result == [True]
    assert np.all(host.numpy() == 7)
    stream.WaitEvent(None)  # null event is a no-op (cuda_stream.cc:160)


def test_single_copies_and_buffers(device):
    buf = device.MakeBuffer()
    n = 12345
    h = buf.MakeHostBuffer(n)
    d = buf.MakeDeviceBuffer(n)
    h2 = buf.MakeHostBuffer(n)
    from ucm_amd.trans import host_view

    host_view(h, n)[:] = rng_for(6).integers(0, 256, size=n, dtype=np.uint8)
    host_view(h2, n)[:] = 0
    for stream in (device.MakeStream(), device.MakeSMStream()):
        stream.HostToDevice(h, d, n)
        stream.DeviceToHostAsync(d, h2, n)
        stream.Synchronized()
        assert np.array_equal(host_view(h2, n), host_view(h, n))
    buf.release()


def test_errors(device):
    from ucm_amd.trans import Device

    with pytest.raises(ValueError):
        Device().Setup(-1)
    with pytest.raises(ValueError):
        Device().Setup(1000)
    ce = device.MakeStream()
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):  # a copy-engine stream cannot read a device-side table
        ce.DeviceToHostGather(t.data_ptr(), t.data_ptr(), 8, 2)
    with pytest.raises(ValueError):
        ce.PagedGatherAsync([t.data_ptr()], [8], [0], t.data_ptr())
    sm = device.MakeSMStream()
    with pytest.raises(ValueError):  # a negative id would be a wild address
        sm.PagedGatherAsync([t.data_ptr()], [8], [0, -1], t.data_ptr())
    with pytest.raises(ValueError):  # beyond the cache's extent
        sm.PagedScatterAsync(t.data_ptr(), [t.data_ptr()], [8], [0, 8], num_cache_blocks=8)
