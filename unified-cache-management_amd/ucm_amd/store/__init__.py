from .base import Task, UcmKVStoreBaseV1  # noqa: F401
from .host_store import HostMemoryStore  # noqa: F401
