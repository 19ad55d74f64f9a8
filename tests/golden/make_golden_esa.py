"""Writes tests/golden/esa_retrieval_ref.npz from the REFERENCE's own ESA retrieval backend.

Run in the build container only (needs oracle/_ref, i.e. `make -C oracle ref`, which compiles
ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp unmodified).  The fixture holds the inputs
(or the PCG64 seed they are drawn from, see `dense_inputs` / `wide_inputs`) and the backend's
outputs (indices and fp32 scores); tests compare the C checker and the HIP library against it.

Cases
  dense    2 requests, 64 candidates each out of 200 rows of dim 128, top-16.
  ragged   3 requests with candidate lists of different length padded with -1 (also in front),
           dim 48, top-5; one submit per row because get_result assumes equal counts.
  wide     1 request, dim 1024 (the shape of the reference's own driver,
           retrieval_worker.py:45-60, scaled down), 300 candidates, top-100.
  ints     small-integer data: every product and partial sum is exact in fp32, so any correct
           implementation must reproduce these scores bit for bit; includes tied scores.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import ref_backend  # noqa: E402


def run_ref(mod, data, query, indexes, k):
    be = mod.RetrievalWorkerBackend(np.ascontiguousarray(data, np.float32), {0: [0]})
    rid = be.submit(np.ascontiguousarray(query, np.float32), int(k), np.ascontiguousarray(indexes, np.int32))
    be.wait(rid)
    r = be.get_result(rid)
    out = (np.array(r["indices"], np.int32), np.array(r["scores"], np.float32))
    del be
    return out


def dense_inputs(seed=5005):
    """Shared with the tests."""
    rng = np.random.Generator(np.random.PCG64(seed))
    data = rng.standard_normal((200, 128)).astype(np.float32)
    query = rng.standard_normal((2, 128)).astype(np.float32)
    indexes = np.stack([rng.permutation(200)[:64] for _ in range(2)]).astype(np.int32)
    return data, query, indexes


def wide_inputs(seed=7007):
    """Shared with the tests."""
    rng = np.random.Generator(np.random.PCG64(seed))
    data = rng.random((400, 1024), dtype=np.float32)
    query = rng.random((1, 1024), dtype=np.float32)
    indexes = rng.permutation(400)[:300].astype(np.int32)[None, :]
    return data, query, indexes


def main():
    mod = ref_backend("retrieval_backend")
    if mod is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref` first")
    out = {}
    data, query, indexes = dense_inputs()
    i, s = run_ref(mod, data, query, indexes, 16)
    out.update(dense_seed=np.int64(5005), dense_indexes=indexes, dense_idx=i, dense_score=s)

    rng = np.random.Generator(np.random.PCG64(6006))
    data = rng.standard_normal((60, 48)).astype(np.float32)
    query = rng.standard_normal((3, 48)).astype(np.float32)
    indexes = -np.ones((3, 20), np.int32)
    indexes[0, :20] = rng.permutation(60)[:20]
    indexes[1, :3] = rng.permutation(60)[:3]
    indexes[2, 4:15] = rng.permutation(60)[:11]
    ii, ss = [], []
    for r in range(3):
        i, s = run_ref(mod, data, query[r:r + 1], indexes[r:r + 1], 5)
        pad = 5 - i.shape[1]
        ii.append(np.pad(i[0], (0, pad), constant_values=-1))
        ss.append(np.pad(s[0], (0, pad), constant_values=0))
    out.update(ragged_data=data, ragged_query=query, ragged_indexes=indexes,
               ragged_idx=np.stack(ii), ragged_score=np.stack(ss))

    data, query, indexes = wide_inputs()
    i, s = run_ref(mod, data, query, indexes, 100)
    out.update(wide_seed=np.int64(7007), wide_indexes=indexes, wide_idx=i, wide_score=s)

    rng = np.random.Generator(np.random.PCG64(8008))
    data = rng.integers(-3, 4, size=(50, 32)).astype(np.float32)
    data[7] = data[21]  # identical rows: tied scores
    query = rng.integers(-3, 4, size=(2, 32)).astype(np.float32)
    indexes = np.tile(np.arange(50, dtype=np.int32), (2, 1))
    i, s = run_ref(mod, data, query, indexes, 50)
    out.update(ints_data=data, ints_query=query, ints_idx=i, ints_score=s)

    path = os.path.join(HERE, "esa_retrieval_ref.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
