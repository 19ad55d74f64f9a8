"""Writes tests/golden/hash_retrieval_ref.npz from the REFERENCE's own CPU backend.

Run in the build container only (needs oracle/_ref, i.e. `make -C oracle ref`, which
compiles ucm/sparse/gsa_on_device/csrc/cuda/hash_retrieval/cpy/hash_retrieval_backend.cpp
unmodified).  The fixture holds inputs (or their seed + sha256 when large) and the
backend's outputs; tests compare the C oracle and the HIP library against it.

Cases
  c1_gqa   BASELINE.json config 1: 1 request, 32 q heads / 8 KV heads, 8192 tokens in 64 blocks of
           128, 128-bit codes, top-16.  The backend has no head or group notion, so the GQA
           group sum is obtained through
               dist(concat_g q_g, tile_G(k)) = sum_g dist(q_g, k)
           i.e. per KV head h: data = k[:, :, h, :] repeated G times along dim, query =
           q[h*G:(h+1)*G] concatenated.  k=16 (the config) and k=64 (full ranking = every
           block score) are both recorded.
  ragged   3 rows with different allowed-block lists padded with -1, dim 16, block 8.
  tail     dim 20 (one 16-byte vector + 4 tail bytes, hash_retrieval_backend.cpp:376-383).
  zero     a row whose query equals a cached token: early exit at score 0 (:385-388).
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import ref_backend  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def run_ref(mod, data_u8, query_u8, indexes, k):
    be = mod.HashRetrievalWorkerBackend(np.ascontiguousarray(data_u8), {0: [0]})
    rid = be.submit(np.ascontiguousarray(query_u8), int(k), np.ascontiguousarray(indexes, np.int32))
    be.wait(rid)
    r = be.get_result(rid)
    out = (np.array(r["indices"], np.int32), np.array(r["scores"], np.int32))
    del be
    return out


def c1_inputs(seed=1001):
    """Shared with the tests: BASELINE.json config 1 inputs from one PCG64 stream."""
    rng = np.random.Generator(np.random.PCG64(seed))
    keys = rng.integers(0, 2**32, size=(64, 128, 8, 4), dtype=np.uint32)
    q = rng.integers(0, 2**32, size=(1, 32, 4), dtype=np.uint32)
    return keys, q


def main():
    mod = ref_backend()
    if mod is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref` first")
    out = {}

    # ---- c1_gqa ----
    keys, q = c1_inputs()
    G = 4
    out["c1_seed"] = np.int64(1001)
    out["c1_keys_sha256"] = np.array(sha(keys))
    out["c1_q_sha256"] = np.array(sha(q))
    idx16, sc16, idx64, sc64 = [], [], [], []
    for h in range(8):
        kh = np.ascontiguousarray(keys[:, :, h, :]).view(np.uint8)  # [64,128,16]
        data = np.tile(kh, (1, 1, G))  # [64,128,64]
        qq = np.ascontiguousarray(q[0, h * G:(h + 1) * G]).view(np.uint8).reshape(1, -1)  # [1,64]
        allowed = np.arange(64, dtype=np.int32).reshape(1, 64)
        i, s = run_ref(mod, data, qq, allowed, 16)
        idx16.append(i[0]); sc16.append(s[0])
        i, s = run_ref(mod, data, qq, allowed, 64)
        idx64.append(i[0]); sc64.append(s[0])
    out["c1_idx16"] = np.stack(idx16); out["c1_dist16"] = np.stack(sc16)
    out["c1_idx64"] = np.stack(idx64); out["c1_dist64"] = np.stack(sc64)

    # ---- ragged ----
    rng = np.random.Generator(np.random.PCG64(2002))
    data = rng.integers(0, 256, size=(40, 8, 16), dtype=np.uint8)
    query = rng.integers(0, 256, size=(3, 16), dtype=np.uint8)
    indexes = -np.ones((3, 24), np.int32)
    indexes[0, :24] = rng.permutation(40)[:24]
    indexes[1, :7] = rng.permutation(40)[:7]
    indexes[2, 2:15] = rng.permutation(40)[:13]  # -1 entries in front are stripped too
    out["ragged_data"] = data; out["ragged_query"] = query; out["ragged_indexes"] = indexes
    # one submit per row so that each row's k can differ from its list length
    for name, k in (("k5", 5), ("k10", 10)):
        ii, ss = [], []
        for r in range(3):
            i, s = run_ref(mod, data, query[r:r + 1], indexes[r:r + 1], k)
            pad = k - i.shape[1]
            ii.append(np.pad(i[0], (0, pad), constant_values=-1))
            ss.append(np.pad(s[0], (0, pad), constant_values=0))
        out[f"ragged_idx_{name}"] = np.stack(ii); out[f"ragged_dist_{name}"] = np.stack(ss)

    # ---- tail ----
    rng = np.random.Generator(np.random.PCG64(3003))
    data = rng.integers(0, 256, size=(12, 4, 20), dtype=np.uint8)
    query = rng.integers(0, 256, size=(2, 20), dtype=np.uint8)
    indexes = np.tile(np.arange(12, dtype=np.int32), (2, 1))
    i, s = run_ref(mod, data, query, indexes, 12)
    out["tail_data"] = data; out["tail_query"] = query
    out["tail_idx"] = i; out["tail_dist"] = s

    # ---- zero ----
    rng = np.random.Generator(np.random.PCG64(4004))
    data = rng.integers(0, 256, size=(6, 4, 16), dtype=np.uint8)
    query = data[3, 2][None, :].copy()
    indexes = np.arange(6, dtype=np.int32)[None, :]
    i, s = run_ref(mod, data, query, indexes, 3)
    out["zero_data"] = data; out["zero_query"] = query
    out["zero_idx"] = i; out["zero_dist"] = s

    path = os.path.join(HERE, "hash_retrieval_ref.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
