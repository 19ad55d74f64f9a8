"""GPU twin of the reference's ESA retrieval backend (float dot-product top-k), same object API.

`RetrievalWorkerBackend(data, cpu_idx_tbl)` / `.submit(query, topk, indexes) -> id` /
`.poll(id)` / `.wait(id)` / `.get_result(id) -> {"indices", "scores"}` follow
ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp:20-250 and its Python wrapper
retrieval_worker.py:12-36: per batch row, every allowed row of `data` (entries of `indexes`
other than -1) is scored with its dot product with the query and the `topk` best are returned
in descending score order.  Here the scoring runs on the MI355X through ucm_dot_topk on a side
stream; equal scores keep list order (the reference leaves ties unspecified), and the fp32
sums are taken in a different order than the reference's sequential loop.
"""
import numpy as np
import torch

from .. import _lib


def dot_topk(data, query, indexes, topk, workspace=None):
    """data fp32 [n, dim], query fp32 [B, dim], indexes int32 [B, max_n] (all on one GPU) ->
    (indices int32 [B, topk], scores fp32 [B, topk]) on torch's current stream."""
    if data.dtype != torch.float32 or query.dtype != torch.float32 or indexes.dtype != torch.int32:
        raise ValueError("data and query must be float32, indexes int32")
    if data.device.type != "cuda" or query.device != data.device or indexes.device != data.device:
        raise ValueError("the HIP library needs all tensors on one GPU device")
    if data.dim() != 2 or query.dim() != 2 or indexes.dim() != 2:
        raise ValueError("data [n,dim], query [B,dim], indexes [B,max_n] expected")
    if query.shape[1] != data.shape[1]:
        raise RuntimeError("Query dim mismatch")
    if indexes.shape[0] != query.shape[0]:
        raise RuntimeError("Query and indexes batch mismatch")
    data, query, indexes = data.contiguous(), query.contiguous(), indexes.contiguous()
    B, max_n = indexes.shape
    k = int(topk)
    out_idx = torch.empty((B, k), dtype=torch.int32, device=data.device)
    out_sc = torch.empty((B, k), dtype=torch.float32, device=data.device)
    if B == 0 or max_n == 0:
        return out_idx.fill_(-1), out_sc.zero_()
    need = _lib.lib().ucm_dot_topk_workspace_bytes(B, max_n)
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=data.device)
    _lib.check(_lib.lib().ucm_dot_topk(
        data.data_ptr(), data.shape[0], data.shape[1], query.data_ptr(), indexes.data_ptr(), B, max_n, k,
        out_idx.data_ptr(), out_sc.data_ptr(), workspace.data_ptr(), workspace.numel(),
        _lib.stream_ptr(data.device)))
    return out_idx, out_sc


class RetrievalWorkerBackend:
    def __init__(self, data, cpu_idx_tbl=None, device="cuda:0"):
        """data: float32 [n_items, dim] (numpy or torch).  cpu_idx_tbl (the reference's
        core-pinning table) is accepted and ignored."""
        t = torch.as_tensor(data)
        if t.dim() != 2:
            raise RuntimeError("data must be [n_items, dim]")
        self.device = torch.device(device)
        self.data = t.to(self.device, dtype=torch.float32).contiguous()
        self.n_items, self.dim = (int(x) for x in t.shape)
        self._stream = torch.cuda.Stream(device=self.device)
        self._next = 0
        self._pending = {}
        self._results = {}

    def submit(self, query, topk, indexes):
        q = torch.as_tensor(query)
        if q.dim() != 2 or q.shape[1] != self.dim:
            raise RuntimeError("Query dim mismatch")
        idx = torch.as_tensor(indexes)
        if idx.dim() != 2 or idx.shape[0] != q.shape[0]:
            raise RuntimeError("Query and indexes batch mismatch")
        counts = (idx != -1).sum(dim=1).cpu().numpy() if idx.numel() else np.zeros(q.shape[0], np.int64)
        req = self._next
        self._next += 1
        with torch.cuda.stream(self._stream):
            qd = q.to(self.device, dtype=torch.float32, non_blocking=True)
            td = idx.to(self.device, dtype=torch.int32, non_blocking=True)
            ii, ss = dot_topk(self.data, qd, td, max(int(topk), 1))
            ev = torch.cuda.Event()
            ev.record(self._stream)
        self._pending[req] = (ev, ii, ss, counts, int(topk))
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
        # the reference sizes the result by the first row's count (retrieval_backend.cpp:134-136)
        n = int(min(k, counts[0])) if len(counts) else 0
        self._results[req_id] = {"indices": ii[:, :n].cpu().numpy(), "scores": ss[:, :n].cpu().numpy()}

    def get_result(self, req_id):
        if req_id in self._pending and self._pending[req_id][0].query():
            self.wait(req_id)
        if req_id not in self._results:
            raise RuntimeError("Result not ready")
        return self._results.pop(req_id)  # consumed once (retrieval_backend.cpp:149)


class RetrievalWorker:
    """retrieval_worker.py:12-36: converts the query to float32 and forwards."""

    def __init__(self, cpp_worker):
        self.cpp_worker = cpp_worker

    @classmethod
    def handle_input(cls, input):
        if input.dtype != torch.float32:
            input = input.to(torch.float32)
        return input

    def submit(self, query, topk, indexes):
        return self.cpp_worker.submit(self.handle_input(query), topk, indexes)

    def poll(self, req_id):
        return self.cpp_worker.poll(req_id)

    def get_result(self, req_id):
        return self.cpp_worker.get_result(req_id)

    def wait(self, req_id):
        return self.cpp_worker.wait(req_id)
