"""ctypes loader of libucm_hip.so and status-to-exception translation."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libucm_hip.so")

UCM_OK = 0
UCM_ERROR = -1
UCM_EPARAM = -50000
UCM_EOOM = -50001
UCM_ERETRY = -50004
UCM_ENOOBJ = -50005
UCM_EUNSUPPORTED = -50008
UCM_ETIMEOUT = -50010

DT_BF16, DT_F16, DT_F32 = 0, 1, 2
TOPK_REDUCE_HEADS, TOPK_RETURN_PHYSICAL, TOPK_SCORE_ORDER, TOPK_DISTANCE = 1, 2, 4, 8
TRANS_CE, TRANS_SM = 0, 1

_lib = None

i32, i64, u32, u64 = C.c_int32, C.c_int64, C.c_uint32, C.c_uint64
vp, sz, ci = C.c_void_p, C.c_size_t, C.c_int

_SIGNATURES = {
    "ucm_version": (ci, []),
    "ucm_last_error": (C.c_char_p, []),
    "ucm_hash_encode": (ci, [vp, ci, i64, i32, i32, i64, i64, vp, ci, i32, i32, i32, vp, i64, i64, vp]),
    "ucm_hash_encode_cache": (ci, [vp, ci, i64, i32, i32, i64, i64, vp, ci, i32, i32, i32, vp, ci,
                                   vp, i64, i32, i64, i64, i64, vp]),
    "ucm_hash_encode_set_stream_threshold": (ci, [i64]),
    "ucm_hash_encode_set_clock_probe": (ci, [vp]),
    "ucm_hash_encode_stream_timeouts": (i64, []),
    "ucm_hash_encode_clear_stream_timeouts": (ci, []),
    "ucm_hash_encode_debug_trip_stream_latch": (ci, []),
    "ucm_hash_encode_paged": (ci, [vp, ci, i64, i32, i32, i32, i64, i64, i64, vp, i64, i64, vp, ci,
                                   i32, i32, i32, vp, i64, i64, i64, i64, vp]),
    "ucm_code_scatter": (ci, [vp, i64, i32, i32, i64, i64, vp, ci, vp, i64, i32, i64, i64, i64, vp]),
    "ucm_hamming_topk_workspace_bytes": (sz, [i32, i32, i32]),
    "ucm_hamming_topk": (ci, [vp, i64, i64, vp, i64, i32, i32, i32, i64, i64, i64, vp, i32, i32,
                              vp, i32, i32, i32, i32, i32, u32, vp, vp, vp, sz, vp]),
    "ucm_hamming_topk_static": (ci, [vp, i64, i64, vp, i64, i32, i32, i32, i64, i64, i64, vp, i32, i32,
                                     vp, i32, i32, i32, i32, i32, u32, vp, vp, vp]),
    "ucm_hamming_topk_set_profile_events": (ci, [vp, vp]),
    "ucm_hamming_topk_set_clock_probe": (ci, [vp]),
    "ucm_hamming_last_dispatch": (i64, [C.c_char_p, sz]),
    "ucm_sparse_decode_step": (ci, [vp, i64, i64, i64, vp, ci, vp, i64, i64, ci, i32, vp, ci, i32, i32,
                                    vp, i64, i32, i32, i64, i64, i64, vp, i32, i32, vp, i32, i32, i32,
                                    i32, i32, u32, vp, vp, vp, vp, sz, vp]),
    "ucm_gsa_decode_step": (ci, [vp, i64, i64, i64, vp, ci, vp, i64, i64, ci, i32, vp, ci, i32, i32,
                                 vp, i64, i32, i32, i64, i64, i64, vp, i32, i32, vp, i32, i32, i32,
                                 i32, i32, i32, vp, vp, i32, vp, vp, sz, vp]),
    "ucm_sparse_decode_step_mla": (ci, [vp, i64, vp, i64, i64, vp, ci, vp, i64, i64, vp, i64, i64, ci, i32, i32,
                                        vp, vp, ci, i32, i32, vp, i64, i32, i64, i64, vp, i32, i32, vp, i32,
                                        i32, i32, i32, i32, u32, vp, vp, vp, vp, sz, vp]),
    "ucm_gsa_decode_step_mla": (ci, [vp, i64, vp, i64, i64, vp, ci, vp, i64, i64, vp, i64, i64, ci, i32, i32,
                                     vp, vp, ci, i32, i32, vp, i64, i32, i64, i64, vp, i32, i32, vp, i32,
                                     i32, i32, i32, i32, i32, i32, vp, vp, i32, vp, vp, sz, vp]),
    "ucm_hamming_score": (ci, [vp, i64, i64, vp, i64, i32, i32, i32, i64, i64, i64, vp, i32, i32,
                               vp, i32, i32, i32, i32, i32, ci, vp, ci, vp, sz, vp]),
    "ucm_hamming_score_workspace_bytes": (sz, [i32, i32, i32]),
    "ucm_update_seq_lens": (ci, [vp, i32, i32, i32, vp, vp]),
    "ucm_trans_setup": (ci, [i32]),
    "ucm_trans_stream_create": (ci, [ci, C.POINTER(vp)]),
    "ucm_trans_stream_destroy": (ci, [vp]),
    "ucm_trans_stream_handle": (vp, [vp]),
    "ucm_trans_stream_sync": (ci, [vp]),
    "ucm_trans_stream_wait_event": (ci, [vp, vp]),
    "ucm_trans_stream_append_callback": (ci, [vp, vp, vp]),
    "ucm_trans_d2h": (ci, [vp, vp, vp, sz, ci]),
    "ucm_trans_h2d": (ci, [vp, vp, vp, sz, ci]),
    "ucm_trans_gather": (ci, [vp, vp, ci, vp, sz, sz, ci]),
    "ucm_trans_scatter": (ci, [vp, vp, vp, ci, sz, sz, ci]),
    "ucm_trans_batch": (ci, [vp, vp, vp, ci, sz, sz, ci]),
    "ucm_trans_paged_copy": (ci, [vp, vp, vp, i32, vp, i64, i64, vp, ci, ci]),
    "ucm_trans_host_alloc": (ci, [sz, C.POINTER(vp)]),
    "ucm_trans_host_free": (ci, [vp]),
    "ucm_trans_device_alloc": (ci, [sz, C.POINTER(vp)]),
    "ucm_trans_device_free": (ci, [vp]),
    "ucm_trans_host_register": (ci, [vp, sz, C.POINTER(vp)]),
    "ucm_trans_host_unregister": (ci, [vp]),
    "ucm_dot_topk_workspace_bytes": (sz, [i32, i32]),
    "ucm_dot_topk": (ci, [vp, i64, i32, vp, vp, i32, i32, i32, vp, vp, vp, sz, vp]),
    "ucm_kvstar_topk_workspace_bytes": (sz, [i32, i32, i64, i32]),
    "ucm_kvstar_topk": (ci, [vp, i32, i32, i32, vp, i64, i32, i32, i32, vp, i32, vp, vp, vp, sz, vp]),
    "ucm_cache_store_create": (ci, [i32, vp, sz, sz, sz, sz, vp, C.POINTER(vp)]),
    "ucm_cache_store_destroy": (ci, [vp]),
    "ucm_cache_store_nodes": (sz, [vp]),
    "ucm_cache_store_lookup": (ci, [vp, vp, sz, vp]),
    "ucm_cache_store_lookup_on_prefix": (ci, [vp, vp, sz, C.POINTER(i64)]),
    "ucm_cache_store_dump": (ci, [vp, vp, vp, vp, sz, vp, C.POINTER(i64)]),
    "ucm_cache_store_load": (ci, [vp, vp, vp, vp, sz, C.POINTER(i64)]),
    "ucm_cache_store_check": (ci, [vp, i64, C.POINTER(ci)]),
    "ucm_cache_store_wait": (ci, [vp, i64]),
    "ucm_posix_store_create": (ci, [vp, C.POINTER(vp)]),
    "ucm_posix_store_destroy": (ci, [vp]),
    "ucm_posix_store_data_file_path": (i64, [vp, vp, i32, C.c_char_p, sz]),
    "ucm_posix_store_commit": (ci, [vp, vp, i32]),
    "ucm_posix_store_lookup_on_prefix": (ci, [vp, vp, sz, C.POINTER(i64)]),
    "ucm_posix_store_lookup": (ci, [vp, vp, sz, vp]),
    "ucm_posix_store_dump": (ci, [vp, vp, vp, vp, sz, C.POINTER(i64)]),
    "ucm_posix_store_load": (ci, [vp, vp, vp, vp, sz, C.POINTER(i64)]),
    "ucm_posix_store_check": (ci, [vp, i64, C.POINTER(i32)]),
    "ucm_posix_store_wait": (ci, [vp, i64]),
    "ucm_posix_store_gc_once": (ci, [vp, C.POINTER(u64)]),
    "ucm_posix_store_backend": (ci, [vp, vp]),
}


class PosixConfig(C.Structure):
    """ucm_posix_config_t"""
    _fields_ = [
        ("storage_backends", C.POINTER(C.c_char_p)), ("n_backends", sz),
        ("device_id", i32), ("io_direct", i32),
        ("tensor_size", sz), ("shard_size", sz), ("block_size", sz),
        ("data_trans_concurrency", sz), ("lookup_concurrency", sz), ("timeout_ms", sz),
        ("data_dir_shard_bytes", sz),
        ("gc_enable", i32), ("reserved", i32), ("capacity_bytes", sz),
        ("gc_recycle_percent", C.c_double), ("gc_trigger_threshold_ratio", C.c_double),
        ("gc_shard_sample_ratio", C.c_double),
        ("gc_max_recycle_count_per_shard", sz), ("gc_check_interval_sec", sz),
    ]


class CacheBackend(C.Structure):
    """ucm_cache_backend_t"""
    LOOKUP = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p)
    MOVE = C.CFUNCTYPE(C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t)
    WAIT = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int64)
    _fields_ = [("ctx", C.c_void_p), ("lookup", LOOKUP), ("dump", MOVE), ("load", MOVE), ("wait", WAIT)]


EXPORTS = tuple(_SIGNATURES)


def lib():
    """The loaded library.  torch is imported first so that the HIP runtime it ships is the one
    the library binds to.  Raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python unified-cache-management_amd/build.py`"
                " (there is no CPU fallback)")
        import torch  # noqa: F401  (loads libamdhip64 before our library resolves it)

        l = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def last_dispatch():
    """Kernels launched by the last top-k / score call on this thread (ucm_hamming_last_dispatch)."""
    buf = C.create_string_buffer(256)
    lib().ucm_hamming_last_dispatch(buf, 256)
    return buf.value.decode()


def last_error():
    return lib().ucm_last_error().decode("utf-8", "replace")


def check(rc):
    """Raise like the reference's bindings do: ValueError for parameter errors,
    NotImplementedError for unsupported cases, RuntimeError otherwise
    (ucm/shared/trans/cpy/trans.py.cc:35-38 turns a failed Status into RuntimeError)."""
    if rc == UCM_OK:
        return
    msg = f"{rc}, {last_error()}"
    if rc == UCM_EPARAM:
        raise ValueError(msg)
    if rc == UCM_EUNSUPPORTED:
        raise NotImplementedError(msg)
    if rc == UCM_EOOM:
        raise MemoryError(msg)
    raise RuntimeError(msg)


def stream_ptr(device=None):
    """hipStream_t of torch's current stream on `device` as an integer."""
    import torch

    return torch.cuda.current_stream(device).cuda_stream


def stride(t, dim):
    """Stride of `dim` in elements; a canonical (dense) value for extent-1 dimensions, whose
    recorded stride is arbitrary."""
    if t.shape[dim] > 1:
        return t.stride(dim)
    n = 1
    for d in range(dim + 1, t.dim()):
        n *= t.shape[d]
    return n
