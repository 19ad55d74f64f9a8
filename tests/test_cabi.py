"""CPU-side checks of the C-ABI boundary: the library loads, exports exactly what
include/ucm_hip.h declares, and the host mirror validates arguments without a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ucm_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ucm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_groups():
    names = declared_symbols()
    for must in ("ucm_hash_encode", "ucm_hash_encode_cache", "ucm_code_scatter", "ucm_hamming_topk",
                 "ucm_hamming_score", "ucm_update_seq_lens", "ucm_trans_gather",
                 "ucm_trans_scatter", "ucm_trans_batch", "ucm_trans_paged_copy"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from ucm_amd import _lib

    lib = _lib.lib()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in ucm_hip.h but not exported"
    # and the Python binding table covers the same set
    assert sorted(_lib.EXPORTS) == declared_symbols()


def test_version_and_error_string():
    from ucm_amd import _lib

    lib = _lib.lib()
    assert lib.ucm_version() >= 100
    assert isinstance(_lib.last_error(), str)


def test_status_codes_follow_the_reference_convention():
    """ucm/shared/infra/status/status.h:40-53: OK 0, error -1, typed -50000-i."""
    text = open(HEADER).read()
    vals = dict(re.findall(r"#define (UCM_[A-Z]+)\s+\(?(-?\d+)\)?", text))
    assert int(vals["UCM_OK"]) == 0 and int(vals["UCM_ERROR"]) == -1
    assert int(vals["UCM_EPARAM"]) == -50000 and int(vals["UCM_EOOM"]) == -50001
    assert int(vals["UCM_EUNSUPPORTED"]) == -50008 and int(vals["UCM_ETIMEOUT"]) == -50010


def test_parameter_errors_need_no_gpu():
    """Argument validation happens before any HIP call."""
    from ucm_amd import _lib

    lib = _lib.lib()
    rc = lib.ucm_hamming_topk(None, 0, 0, None, 0, 0, 0, 0, 0, 0, 0, None, 0, 0, None, 1, 1, 1, 0,
                              0, 0, None, None, None, 0, None)
    assert rc == _lib.UCM_EPARAM and "null" in _lib.last_error()
    rc = lib.ucm_hash_encode(None, 0, 1, 1, 128, 128, 128, None, 0, 1, 0, 128, None, 4, 4, None)
    assert rc == _lib.UCM_EPARAM
    assert lib.ucm_hamming_topk_workspace_bytes(32, 8, 256) >= 32 * 8 * 256 * 4
    # block ids that would turn into wild device addresses are refused before any launch
    base = (ctypes.c_uint64 * 1)(4096)
    size = (ctypes.c_uint64 * 1)(64)
    flat = ctypes.c_void_p(4096)
    for ids, n_cache in (((ctypes.c_int32 * 2)(0, -1), 0), ((ctypes.c_int32 * 2)(1, 9), 9)):
        rc2 = lib.ucm_trans_paged_copy(None, base, size, 1, ids, 2, n_cache, flat, 0, 0)
        assert rc2 == _lib.UCM_EPARAM and "block_ids[1]" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)


def test_host_mirror_rejects_cpu_tensors():
    import torch

    from ucm_amd.sparse import HashEncoder, hamming_topk

    enc = HashEncoder(128, 128, torch.float32, torch.device("cpu"))
    with pytest.raises(ValueError):
        enc.compute_hash(torch.zeros(2, 128))
    q = torch.zeros(1, 8, 4, dtype=torch.int32)
    k = torch.zeros(2, 16, 8, 4, dtype=torch.int32)
    with pytest.raises(ValueError):
        hamming_topk(q, k, torch.zeros(1, 2, dtype=torch.int32), torch.zeros(1, dtype=torch.int32), 1)


def test_no_product_code_touches_the_oracle():
    """The shipped package must never import the CPU checker."""
    pkg = os.path.join(ROOT, "unified-cache-management_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "README.md", f


def test_encoder_timeout_latch_refuses_further_encodes_until_cleared():
    """A streaming encode whose bounded LDS wait gave up leaves undefined codes behind; from then on
    every encode entry point on that device must fail with UCM_ERROR and say why, before it touches
    the device, until the caller acknowledges.  The latch is tripped from the host here (what a
    timed-out wave does from the device), so the whole error path runs without a GPU."""
    import numpy as np

    from ucm_amd import _lib

    lib = _lib.lib()
    x = np.zeros((4, 1, 128), np.uint16)
    w = np.zeros((128, 128), np.uint16)
    out = np.zeros((4, 1, 4), np.uint32)
    cache = np.zeros((1, 4, 1, 4), np.uint32)
    slots = np.arange(4, dtype=np.int32)

    def encode():
        return lib.ucm_hash_encode(x.ctypes.data, _lib.DT_BF16, 4, 1, 128, 128, 128, w.ctypes.data, _lib.DT_BF16,
                                   1, 1, 128, out.ctypes.data, 4, 4, None)

    def encode_cache():
        return lib.ucm_hash_encode_cache(x.ctypes.data, _lib.DT_BF16, 4, 1, 128, 128, 128, w.ctypes.data,
                                         _lib.DT_BF16, 1, 1, 128, slots.ctypes.data, 0, cache.ctypes.data,
                                         1, 4, 16, 4, 4, None)

    assert lib.ucm_hash_encode_clear_stream_timeouts() == _lib.UCM_OK
    try:
        assert lib.ucm_hash_encode_debug_trip_stream_latch() == _lib.UCM_OK
        for call in (encode, encode_cache):
            assert call() == _lib.UCM_ERROR
            msg = _lib.last_error()
            assert "gave up waiting" in msg and "ucm_hash_encode_clear_stream_timeouts" in msg
        # sticky: a second call fails the same way
        assert encode() == _lib.UCM_ERROR
    finally:
        assert lib.ucm_hash_encode_clear_stream_timeouts() == _lib.UCM_OK
    # acknowledged: the call gets past the latch (whatever it returns without a GPU, it is not the latch)
    encode()
    assert "gave up waiting" not in _lib.last_error()


def test_torch_operator_library_registers_its_operators():
    """torch.ops.ucm_amd.* (the TORCH_LIBRARY registration over the C ABI) loads without a GPU and
    carries the three operators; a CPU tensor has no kernel behind it and is refused by the dispatcher."""
    import torch

    from ucm_amd import torch_ops

    ops = torch_ops.load()
    for name in ("hash_encode_cache", "hamming_topk", "gsa_decode_step"):
        assert hasattr(ops, name)
    z = torch.zeros((1, 1, 4), dtype=torch.int32)
    with pytest.raises((NotImplementedError, RuntimeError)):
        ops.hamming_topk(z, z.view(1, 1, 1, 4), z.view(1, 4)[:, :1], z.view(-1)[:1], 1, 0, 0, 0)
