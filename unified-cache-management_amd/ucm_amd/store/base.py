"""Signatures of the reference's KV store interface (ucm/store/ucmstore_v1.py:41-204), kept so
that connectors and retrieval plugins reach the MI355X transfer path the way they reach any
UCM store.  Only the interface is mirrored; the reference's store stack is not rebuilt."""
from abc import ABC, abstractmethod
from typing import Dict, List

import numpy as np


class Task(ABC):
    """Opaque handle of an asynchronous transfer."""


class UcmKVStoreBaseV1(ABC):
    def __init__(self, config: Dict[str, object]) -> None:
        self.config = config

    @abstractmethod
    def cc_store(self) -> int: ...

    @abstractmethod
    def lookup(self, block_ids: List[bytes]) -> List[bool]: ...

    @abstractmethod
    def lookup_on_prefix(self, block_ids: List[bytes]) -> int: ...

    @abstractmethod
    def prefetch(self, block_ids: List[bytes]) -> None: ...

    @abstractmethod
    def load(self, block_ids: List[bytes], shard_index: List[int], dst_tensor) -> Task: ...

    @abstractmethod
    def dump(self, block_ids: List[bytes], shard_index: List[int], src_tensor) -> Task: ...

    @abstractmethod
    def load_data(self, block_ids: List[bytes], shard_index: List[int],
                  dst_addr: "List[List[int]] | np.ndarray") -> Task: ...

    @abstractmethod
    def dump_data(self, block_ids: List[bytes], shard_index: List[int],
                  src_addr: "List[List[int]] | np.ndarray", prerequisite_handle: int = 0) -> Task: ...

    @abstractmethod
    def wait(self, task: Task) -> None: ...

    @abstractmethod
    def check(self, task: Task) -> bool: ...
