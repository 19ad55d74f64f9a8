"""torch.ops.ucm_amd.*: the C ABI's operators registered with PyTorch's dispatcher.

    from ucm_amd import torch_ops
    torch_ops.load()
    idx, score = torch.ops.ucm_amd.hamming_topk(q_codes, k_cache, block_table, seq_lens, k, 0, 0, 0)

Counterpart of the reference's torch registration of its NPU operator
(ucm/sparse/gsa_on_device/csrc/ascend/torch_binding.cpp:39-79).  The operators forward raw
pointers to libucm_hip.so; there is no fallback: loading fails when the library is missing.
"""
import os

import torch

from . import _lib

OPS_PATH = os.path.join(os.path.dirname(_lib.LIB_PATH), "libucm_torch_ops.so")
_loaded = False


def load():
    """Registers the operators (once per process) and returns torch.ops.ucm_amd."""
    global _loaded
    if not _loaded:
        if not os.path.exists(OPS_PATH):
            raise RuntimeError(f"{OPS_PATH} is missing: run unified-cache-management_amd/build.py")
        _lib.lib()  # libucm_hip.so first, so that the registration library binds to the loaded one
        torch.ops.load_library(OPS_PATH)
        _loaded = True
    return torch.ops.ucm_amd
