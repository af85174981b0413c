"""Two-tier chunk store: a local store that answers first and a remote store that keeps
everything (LMCache/lmcache/storage_backend/hybrid_backend.py:22-121 in the reference).

Writes go through to both tiers; a read that the local tier cannot serve is answered by the
remote tier and remembered locally.  At start-up the local tier is filled with every chunk the
remote side already holds for this model, world size and worker."""
import logging
from typing import Iterable, List, Optional

import torch

from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from ..utils import CacheEngineKey
from .abstract_backend import LMCBackendInterface
from .local_backend import LMCLocalBackend
from .remote_backend import LMCPipelinedRemoteBackend, LMCRemoteBackend

logger = logging.getLogger("cachegen_amd")


class LMCHybridBackend(LMCBackendInterface):
    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
        remote_cls = LMCPipelinedRemoteBackend if config.pipelined_backend else LMCRemoteBackend
        self.local_store = LMCLocalBackend(config)
        self.remote_store = remote_cls(config, metadata)
        owner = (metadata.model_name, metadata.world_size, metadata.worker_id)
        mine = [k for k in self.remote_store.list() if (k.model_name, k.world_size, k.worker_id) == owner]
        fetched = sum(self._remember(k, self.remote_store.get(k)) for k in mine)
        logger.info("Pre-fetched %d of %d keys from the remote store", fetched, len(mine))

    def _remember(self, key: CacheEngineKey, value: Optional[torch.Tensor]) -> bool:
        """Keeps a chunk that came from the remote tier in the local one."""
        if value is None:
            return False
        self.local_store.put(key, value)
        return True

    def contains(self, key: CacheEngineKey) -> bool:
        return self.local_store.contains(key) or self.remote_store.contains(key)

    def put(self, key: CacheEngineKey, value: torch.Tensor, blocking: bool = True) -> None:
        # the local tier is memory: nothing to wait for, so it is always written at once
        self.local_store.put(key, value, blocking=True)
        self.remote_store.put(key, value, blocking)

    def put_chunks(self, keys, blob, chunk_size, fmt, blocking=True) -> int:
        self.local_store.put_chunks(keys, blob, chunk_size, fmt, blocking=True)
        return self.remote_store.put_chunks(keys, blob, chunk_size, fmt, blocking)

    def get(self, key: CacheEngineKey) -> Optional[torch.Tensor]:
        hit = self.local_store.get(key)
        if hit is not None:
            return hit
        value = self.remote_store.get(key)
        self._remember(key, value)
        return value

    def batched_get(self, keys: Iterable[CacheEngineKey]) -> List[Optional[torch.Tensor]]:
        """Local hits first; all misses go to the remote tier in one batched request."""
        keys = list(keys)
        found = {i: v for i, v in enumerate(map(self.local_store.get, keys)) if v is not None}
        missing = [i for i in range(len(keys)) if i not in found]
        for i, value in zip(missing, self.remote_store.batched_get(keys[i] for i in missing)):
            if self._remember(keys[i], value):
                found[i] = value
        return [found.get(i) for i in range(len(keys))]

    def close(self):
        for tier in (self.local_store, self.remote_store):
            tier.close()
