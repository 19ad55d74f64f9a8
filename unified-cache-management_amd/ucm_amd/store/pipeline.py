"""Store pipelines by name, as the reference builds them.

`UcmPipelineStore(config)` reads `config["store_pipeline"]` and stacks the native stores the way
ucm/store/pipeline/connector.py:160-217 stacks the reference's libraries:

    "Posix"        one PosixStore
    "Cache"        one CacheStore (pinned staging only)
    "Cache|Posix"  a CacheStore whose backend is a PosixStore configured with
                   tensor_size = shard_size, exactly as connector.py:180-188 does

Every method of the store interface goes to the front store of the stack.
"""
import copy
from typing import Dict

from .base import UcmKVStoreBaseV1
from .cache_store import CacheStore
from .posix_store import PosixStore


def _posix(config):
    return [PosixStore(config)]


def _cache(config):
    return [CacheStore(config)]


def _cache_posix(config):
    posix_config = copy.copy(config)
    if int(config.get("device_id", -1)) >= 0:
        posix_config["tensor_size"] = config["shard_size"]
    posix = PosixStore(posix_config)
    if int(config.get("device_id", -1)) < 0:
        return [posix]  # the lookup-only side needs no staging buffer in front
    cache_config = copy.copy(config)
    cache_config["store_backend"] = posix
    return [posix, CacheStore(cache_config)]


_BUILDERS = {"Posix": _posix, "Cache": _cache, "Cache|Posix": _cache_posix}


class UcmPipelineStore(UcmKVStoreBaseV1):
    def __init__(self, config: Dict[str, object]) -> None:
        super().__init__(config)
        name = config.get("store_pipeline")
        if name not in _BUILDERS:
            raise ValueError(f"unknown store pipeline: {name}")
        self._stores = _BUILDERS[name](config)
        self._front = self._stores[-1]

    def close(self):
        for s in reversed(self._stores):
            s.close()
        self._stores = []

    def cc_store(self):
        return self._front.cc_store()

    def lookup(self, block_ids):
        return self._front.lookup(block_ids)

    def lookup_on_prefix(self, block_ids):
        return self._front.lookup_on_prefix(block_ids)

    def prefetch(self, block_ids):
        return self._front.prefetch(block_ids)

    def load(self, block_ids, shard_index, dst_tensor):
        return self._front.load(block_ids, shard_index, dst_tensor)

    def dump(self, block_ids, shard_index, src_tensor):
        return self._front.dump(block_ids, shard_index, src_tensor)

    def load_data(self, block_ids, shard_index, dst_addr):
        return self._front.load_data(block_ids, shard_index, dst_addr)

    def dump_data(self, block_ids, shard_index, src_addr, prerequisite_handle=0):
        return self._front.dump_data(block_ids, shard_index, src_addr, prerequisite_handle)

    def wait(self, task):
        return self._front.wait(task)

    def check(self, task):
        return self._front.check(task)
