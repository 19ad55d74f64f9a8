"""MI355X-native sparse-retrieval and KV-transfer hot path behind UCM's operator surface.

The package is a thin host-side mirror of the reference's operator interfaces
(HashEncoder, cuda_hamming_topk / hamming_score, HashRetrievalWorker, ucmtrans Device/Stream)
over the C-ABI library libucm_hip.so.  There is no CPU fallback: every operator raises if the
library cannot be loaded.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
