from .base import Task, UcmKVStoreBaseV1  # noqa: F401
from .host_store import HostMemoryStore  # noqa: F401
from .cache_store import CacheStore  # noqa: F401
from .posix_store import PosixStore  # noqa: F401
from .pipeline import UcmPipelineStore  # noqa: F401
