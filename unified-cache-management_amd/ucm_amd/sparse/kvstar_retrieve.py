"""GPU twin of the reference's KVStar retrieval library, same module-level API.

The reference binds `Setup`, `AsyncRetrieveByCPU`, `Wait`, `GetTaskResult`, `SetupParam` and
`DeviceType` (ucm/sparse/kvstar/retrieve/py_intf/py_intf.cpp:18-112) over a CPU thread pool
whose kernel (core/domain/retrieve_task/simd_compute_kernel.cpp:816-985) scores every KV block
of a request by the attention-probability mass its representatives receive from a group of
recent queries, and returns the `topK` best block numbers.  Here the same quantities are
computed on the MI355X by ucm_kvstar_topk on a side stream; a task id stands for a recorded
event instead of a pool job.  Call sites read like the reference's
(ucm/sparse/kvstar/multistep.py:251-276 submit, :433-446 wait and fetch):

    task_id = kvstar_retrieve.AsyncRetrieveByCPU(query_group, blk_repre, d_pruned_index,
                                                 topk, req_id, kvstar_retrieve.CPU)
    kvstar_retrieve.Wait(task_id)
    result = kvstar_retrieve.GetTaskResult(task_id)   # {"status": "SUCCESS", "data": [...]}

Differences from the reference, both confined to inputs with exactly equal block scores or
sums within rounding: equal scores are returned in ascending block order (the reference's heap
yields descending block order and, after a replacement, may keep a later block over an earlier
one), and fp32 sums are taken in a different order.
"""
import enum
import threading
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .. import _lib


class DeviceType(enum.IntEnum):
    CPU = 0
    GPU = 1


CPU = DeviceType.CPU
GPU = DeviceType.GPU


@dataclass
class SetupParam:
    """py_intf.cpp:94-104.  The NUMA and core-binding fields configure the reference's thread
    pool; they are kept for the call sites and have no effect on the GPU path."""
    cpuNumaIds: List[int] = field(default_factory=list)
    bindInfo: List[Tuple[int, int]] = field(default_factory=list)
    deviceType: DeviceType = DeviceType.CPU
    totalTpSize: int = 1
    localRankId: int = 0
    device: Optional[str] = None  # GPU that scores; default cuda:0


def kvstar_topk(query_group, blk_repre, pruned_index, topk, workspace=None):
    """query_group fp16 [x, Hq, d_orig], blk_repre fp16 [n, M, Hkv, d], pruned_index int64
    [Hkv, d] or None, all on one GPU -> (block numbers int32 [min(topk, n)], scores fp32) on
    torch's current stream."""
    if query_group.dtype != torch.float16 or blk_repre.dtype != torch.float16:
        raise ValueError("query_group and blk_repre must be float16")
    if query_group.device.type != "cuda" or blk_repre.device != query_group.device:
        raise ValueError("the HIP library needs all tensors on one GPU device")
    if query_group.dim() != 3:
        raise RuntimeError("Query shape must be 3D (x, H, d).")
    if blk_repre.dim() != 4:
        raise RuntimeError("BlockRep shape must be 4D (n, M, h, d).")
    q, k = query_group.contiguous(), blk_repre.contiguous()
    X, Hq, d_orig = q.shape
    n, M, Hkv, d = k.shape
    pr = None
    if pruned_index is not None:
        if pruned_index.dtype != torch.int64 or tuple(pruned_index.shape) != (Hkv, d):
            raise RuntimeError("dPrunedIndex must be int64 [h, d_pruned]")
        # entries are not range-checked here (that would wait for the GPU); the kernel clamps
        # them into [0, d_orig) so a bad index cannot read outside the query row
        pr = pruned_index.to(q.device).contiguous()
    kk = min(int(topk), n)
    out_idx = torch.empty(max(kk, 1), dtype=torch.int32, device=q.device)
    out_sc = torch.empty(max(kk, 1), dtype=torch.float32, device=q.device)
    if kk <= 0:
        return out_idx[:0], out_sc[:0]
    need = _lib.lib().ucm_kvstar_topk_workspace_bytes(X, Hq, n, M)
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    _lib.check(_lib.lib().ucm_kvstar_topk(
        q.data_ptr(), X, Hq, d_orig, k.data_ptr(), n, M, Hkv, d,
        pr.data_ptr() if pr is not None else None, kk, out_idx.data_ptr(), out_sc.data_ptr(),
        workspace.data_ptr(), workspace.numel(), _lib.stream_ptr(q.device)))
    return out_idx[:kk], out_sc[:kk]


class _Manager:
    def __init__(self):
        self.lock = threading.Lock()
        self.device = None
        self.stream = None
        self.next_id = 1
        self.tasks: Dict[int, dict] = {}

    def setup(self, device):
        with self.lock:
            self.device = torch.device(device or "cuda:0")
            self.stream = torch.cuda.Stream(device=self.device)

    def ensure(self):
        if self.stream is None:
            self.setup(None)


_mgr = _Manager()


def Setup(param: SetupParam) -> int:
    """kvstar_retrieve.cpp Setup: prepares the worker side.  Returns 0 like the reference."""
    _mgr.setup(getattr(param, "device", None))
    return 0


def AsyncRetrieveByCPU(queryGroup, blkRepre, dPrunedIndex, topK, reqId, deviceType) -> int:
    """py_intf.cpp:18-53.  Tensors may live on the host (as at the reference's call site) or
    already on the GPU (no copy then).  A failure while submitting is recorded on the task, as
    the reference's worker records an exception (retrieve_task_runner: status FAILURE)."""
    _mgr.ensure()
    with _mgr.lock:
        tid = _mgr.next_id
        _mgr.next_id += 1
    rec = {"status": "RUNNING", "req": int(reqId)}
    try:
        with torch.cuda.stream(_mgr.stream):
            q = queryGroup.to(_mgr.device, non_blocking=True)
            k = blkRepre.to(_mgr.device, non_blocking=True)
            pr = dPrunedIndex.to(_mgr.device, non_blocking=True) if dPrunedIndex is not None else None
            idx, sc = kvstar_topk(q, k, pr, int(topK))
            ev = torch.cuda.Event()
            ev.record(_mgr.stream)
        rec.update(event=ev, idx=idx, score=sc, keep=(q, k, pr))
    except Exception as e:  # noqa: BLE001 - reported through the task, like the reference
        rec.update(status="FAILURE", error=str(e))
    with _mgr.lock:
        _mgr.tasks[tid] = rec
    return tid


def _finish(rec):
    if rec["status"] == "RUNNING":
        rec["event"].synchronize()
        rec["data"] = [int(v) for v in rec["idx"].cpu().tolist()]
        rec["scores"] = rec["score"].cpu().tolist()
        rec["status"] = "SUCCESS"
        for key in ("event", "idx", "score", "keep"):
            rec.pop(key, None)


def Wait(taskId: int) -> int:
    """retrieve_task_manager.cpp:60-75: blocks until the task has finished; 0 on success,
    non-zero for a failed task, an unknown id or an id already waited for (the reference drops
    the waiter on the first Wait)."""
    with _mgr.lock:
        rec = _mgr.tasks.get(int(taskId))
        if rec is None or rec.get("waited"):
            return 1
        rec["waited"] = True
    _finish(rec)
    return 0 if rec["status"] == "SUCCESS" else 1


def GetTaskResult(taskId: int):
    """py_intf.cpp:55-86: None for an unknown id, else a dict with "status" and, by status,
    "data" (block numbers, best first) or "error"."""
    with _mgr.lock:
        rec = _mgr.tasks.get(int(taskId))
    if rec is None:
        return None
    if rec["status"] == "RUNNING" and rec["event"].query():
        _finish(rec)
    out = {"status": rec["status"]}
    if rec["status"] == "SUCCESS":
        out["data"] = list(rec["data"])
        out["scores"] = list(rec["scores"])
    elif rec["status"] == "FAILURE":
        out["error"] = rec["error"]
    return out
