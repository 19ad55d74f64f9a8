"""GPU twin of the reference's CPU hash-retrieval backend, same object API.

`HashRetrievalWorkerBackend(data, cpu_idx_tbl)` / `.submit(query, topk, indexes) -> id` /
`.poll(id)` / `.wait(id)` / `.get_result(id) -> {"indices", "scores"}` follow
ucm/sparse/gsa_on_device/csrc/cuda/hash_retrieval/cpy/hash_retrieval_backend.cpp:165-444 and its
Python wrapper hash_retrieval_worker.py:12-36: per batch row, every allowed block (entries of
`indexes` other than -1) is scored with the minimum over its block_size tokens of
popcount(query xor key) over `dim` bytes, and the `topk` smallest scores are returned in
ascending score order.  Here the scoring runs on the MI355X through ucm_hamming_topk
(UCM_TOPK_SCORE_ORDER | UCM_TOPK_DISTANCE | UCM_TOPK_RETURN_PHYSICAL) on a side stream;
ties go to the entry that comes first in the row's list (the reference leaves them unspecified).
"""
import numpy as np
import torch

from .hamming_topk import hamming_topk


class HashRetrievalWorkerBackend:
    def __init__(self, data, cpu_idx_tbl=None, device="cuda:0"):
        """data: uint8 [num_blocks, block_size, dim] (numpy or torch); dim % 4 == 0.
        cpu_idx_tbl (the reference's core-pinning table) is accepted and ignored."""
        t = torch.as_tensor(data)
        if t.dtype != torch.uint8 or t.dim() != 3:
            raise RuntimeError("data must be uint8 [num_blocks, block_size, dim]")
        if t.shape[2] % 4:
            raise RuntimeError("dim must be a multiple of 4 bytes")
        self.device = torch.device(device)
        self.data = t.to(self.device).contiguous()
        self.num_blocks, self.block_size, self.dim = (int(x) for x in t.shape)
        self._codes = self.data.view(torch.int32).view(self.num_blocks, self.block_size, 1, self.dim // 4)
        self._stream = torch.cuda.Stream(device=self.device)
        self._next = 0
        self._pending = {}
        self._results = {}

    def submit(self, query, topk, indexes):
        q = torch.as_tensor(query)
        if q.dtype != torch.uint8:
            q = q.to(torch.uint8)
        if q.dim() != 2 or q.shape[1] != self.dim:
            raise RuntimeError("Query dim mismatch")
        idx = np.asarray(indexes.cpu() if isinstance(indexes, torch.Tensor) else indexes, dtype=np.int32)
        if idx.ndim != 2 or idx.shape[0] != q.shape[0]:
            raise RuntimeError("Query and indexes batch mismatch")
        B = q.shape[0]
        # strip -1 entries, keeping order (hash_retrieval_backend.cpp:241-246)
        rows = [r[r != -1] for r in idx]
        counts = np.array([len(r) for r in rows], np.int32)
        width = max(int(counts.max()) if B else 0, 1)
        table = np.zeros((B, width), np.int32)
        for b, r in enumerate(rows):
            table[b, : len(r)] = r
        k = int(topk)
        req = self._next
        self._next += 1
        with torch.cuda.stream(self._stream):
            qd = q.to(self.device, non_blocking=True).contiguous().view(torch.int32).view(B, 1, self.dim // 4)
            td = torch.from_numpy(table).to(self.device, non_blocking=True)
            ld = torch.from_numpy(counts * self.block_size).to(self.device, non_blocking=True)
            ii, ss = hamming_topk(qd, self._codes, td, ld, max(k, 1), score_order=True, distance=True,
                                  return_physical=True)
            ev = torch.cuda.Event()
            ev.record(self._stream)
        self._pending[req] = (ev, ii, ss, counts, k)
        return req

    def poll(self, req_id):
        if req_id in self._results:
            return True
        if req_id not in self._pending:
            return False
        return self._pending[req_id][0].query()

    def wait(self, req_id):
        if req_id in self._results:
            return
        if req_id not in self._pending:
            raise RuntimeError("Bad req_id")
        ev, ii, ss, counts, k = self._pending.pop(req_id)
        ev.synchronize()
        n = int(min(k, counts.max())) if len(counts) else 0
        self._results[req_id] = {"indices": ii[:, 0, :n].cpu().numpy(), "scores": ss[:, 0, :n].cpu().numpy()}

    def get_result(self, req_id):
        if req_id in self._pending and self._pending[req_id][0].query():
            self.wait(req_id)
        if req_id not in self._results:
            raise RuntimeError("Result not ready")
        return self._results.pop(req_id)  # consumed once (hash_retrieval_backend.cpp:298)


class HashRetrievalWorker:
    """hash_retrieval_worker.py:12-36."""

    def __init__(self, cpp_worker):
        self.cpp_worker = cpp_worker

    @classmethod
    def handle_input(cls, input):
        if input.dtype != torch.uint8:
            input = input.to(torch.uint8)
        return input

    def submit(self, query, topk, indexes):
        return self.cpp_worker.submit(self.handle_input(query), topk, indexes)

    def poll(self, req_id):
        return self.cpp_worker.poll(req_id)

    def get_result(self, req_id):
        return self.cpp_worker.get_result(req_id)

    def wait(self, req_id):
        return self.cpp_worker.wait(req_id)
