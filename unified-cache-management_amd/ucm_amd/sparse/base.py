"""Dependency-free mirror of the reference's sparse-attention plugin surface.

Hook names, argument order and defaults follow `UcmSparseBase`
(ucm/sparse/base.py:127-322), the registry follows `UcmSparseFactory`
(ucm/sparse/factory.py:16-56) and the process-global agent follows ucm/sparse/state.py:26-74 —
without importing vLLM, so retrieval plugins written against the reference can subclass this
and reach the MI355X operators.  Engine types (VllmConfig, ForwardContext, SchedulerOutput ...)
are duck-typed.
"""
import enum
import importlib
from abc import ABC, abstractmethod
from typing import Callable, Dict, List, Optional, Tuple, Union


class UcmSparseRole(enum.Enum):
    SCHEDULER = 0
    WORKER = 1


class UcmSparseMetadata(ABC):
    """Opaque per-step metadata passed from the scheduler side to the worker side."""


class UcmSparseBase(ABC):
    def __init__(self, vllm_config, role: UcmSparseRole):
        self._sparse_metadata: Optional[UcmSparseMetadata] = None
        self._vllm_config = vllm_config
        self._role = role

    @property
    def role(self) -> UcmSparseRole:
        return self._role

    # ---- worker side ----
    def bind_sparse_metadata(self, sparse_metadata: UcmSparseMetadata) -> None:
        self._sparse_metadata = sparse_metadata

    def clear_sparse_metadata(self) -> None:
        self._sparse_metadata = None

    def _get_sparse_metadata(self) -> UcmSparseMetadata:
        assert self._sparse_metadata is not None
        return self._sparse_metadata

    def register_kv_caches(self, kv_caches: dict):
        pass

    def execute_begin(self, scheduler_output):
        pass

    def execute_finished(self, logits_indices):
        return logits_indices

    def attention_begin(self, query, key, value, layer_name: str, forward_context, output=None,
                        phase: Optional[str] = None, k_hash=None, decode_ql_nope=None,
                        decode_q_pe=None) -> Tuple:
        return query, key, value, output

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context,
                           phase: Optional[str] = None) -> None:
        pass

    def update_states(self, scheduler_output) -> None:
        pass

    def ffn_begin(self, hidden_states, residual):
        return hidden_states, residual

    def ffn_finished(self, hidden_states, residual):
        return hidden_states, residual

    def layer_begin(self, positions, hidden_states, residual):
        return positions, hidden_states, residual

    def layer_finished(self, positions, hidden_states, residual):
        return positions, hidden_states, residual

    def request_finished_in_worker(self, request_id: Union[int, str]):
        pass

    # ---- scheduler side ----
    @abstractmethod
    def request_begin(self, request_id: Union[int, str], prompt_token_ids: List[int]):
        pass

    def request_finished_in_scheduler(self, request_id: Union[int, str]):
        pass

    def estimate_num_slots_sparsed(self, request) -> int:
        pass

    def update_state_after_alloc(self, request, num_blocks: int):
        pass

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata):
        pass

    def allocate_slots(self, kv_cache_manager, request, num_slots_sparsed):
        pass


class UcmSparseFactory:
    _registry: Dict[str, Callable[[], type]] = {}

    @classmethod
    def register_sparse_method(cls, name: str, module_path: str, class_name: str) -> None:
        if name in cls._registry:
            raise ValueError(f"Sparse attention method '{name}' is already registered.")

        def loader() -> type:
            return getattr(importlib.import_module(module_path), class_name)

        cls._registry[name] = loader

    @classmethod
    def create_sparse_method(cls, config, role: UcmSparseRole, name: Optional[str] = None):
        """`config` carries `ucm_sparse_config: {"<Method>": {...}}`
        (ucm/sparse/factory.py:34-44); the first key picks the plugin unless `name` is given."""
        if name is None:
            sparse_cfg = getattr(config, "ucm_sparse_config", None) or config["ucm_sparse_config"]
            name = next(iter(sparse_cfg))
        if name not in cls._registry:
            raise ValueError(f"Unsupported sparse method: {name}")
        return cls._registry[name]()(config, role)


UcmSparseFactory.register_sparse_method("GSAOnDevice", "ucm_amd.sparse.gsa_on_device", "GSAOnDevice")

_UCM_SPARSE_AGENT: Optional[UcmSparseBase] = None


def ensure_ucm_sparse_initialized(config, role: UcmSparseRole) -> None:
    global _UCM_SPARSE_AGENT
    if _UCM_SPARSE_AGENT is None:
        _UCM_SPARSE_AGENT = UcmSparseFactory.create_sparse_method(config, role)


def has_ucm_sparse() -> bool:
    return _UCM_SPARSE_AGENT is not None


def get_ucm_sparse() -> UcmSparseBase:
    assert _UCM_SPARSE_AGENT is not None, "UCM sparse is not initialized"
    return _UCM_SPARSE_AGENT


def reset_ucm_sparse() -> None:
    global _UCM_SPARSE_AGENT
    _UCM_SPARSE_AGENT = None
