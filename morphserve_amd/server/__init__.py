"""Host-side policy that decides when the KV pool grows, shrinks or evicts."""
from .scheduler import Request, RequestIdManager, Scheduler  # noqa: F401
from .memory_utils import (PoolEngine, org2quant_and_update_kvcache,  # noqa: F401
                           quant2org_and_update_kvcache, update_kvcache_after_replacing_layer)
