"""Local store in front of a remote one: writes go to both, reads fill the local store
(LMCache/lmcache/storage_backend/hybrid_backend.py:22-121)."""
import logging
from typing import Iterable, Optional

import torch

from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from ..utils import CacheEngineKey
from .abstract_backend import LMCBackendInterface
from .local_backend import LMCLocalBackend
from .remote_backend import LMCPipelinedRemoteBackend, LMCRemoteBackend

logger = logging.getLogger("cachegen_amd")


class LMCHybridBackend(LMCBackendInterface):
    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
        self.local_store = LMCLocalBackend(config)
        remote = LMCPipelinedRemoteBackend if config.pipelined_backend else LMCRemoteBackend
        self.remote_store = remote(config, metadata)
        self._prefetch(metadata)

    def _prefetch(self, metadata: LMCacheEngineMetadata) -> None:
        """Pulls every chunk of this model and worker that the remote side already holds."""
        nfetched = 0
        for key in self.remote_store.list():
            if (key.model_name, key.worker_id, key.world_size) != \
                    (metadata.model_name, metadata.worker_id, metadata.world_size):
                continue
            data = self.remote_store.get(key)
            if data is not None:
                self.local_store.put(key, data)
                nfetched += 1
        logger.info("Pre-fetched %d keys from remote backend", nfetched)

    def contains(self, key: CacheEngineKey) -> bool:
        return self.local_store.contains(key) or self.remote_store.contains(key)

    def put(self, key: CacheEngineKey, value: torch.Tensor, blocking: bool = True) -> None:
        self.local_store.put(key, value, blocking=True)
        self.remote_store.put(key, value, blocking)

    def put_chunks(self, keys, blob, chunk_size, fmt, blocking=True) -> int:
        self.local_store.put_chunks(keys, blob, chunk_size, fmt, blocking=True)
        return self.remote_store.put_chunks(keys, blob, chunk_size, fmt, blocking)

    def get(self, key: CacheEngineKey) -> Optional[torch.Tensor]:
        value = self.local_store.get(key)
        if value is None:
            value = self.remote_store.get(key)
            if value is not None:
                self.local_store.put(key, value)
        return value

    def batched_get(self, keys: Iterable[CacheEngineKey]):
        keys = list(keys)
        ret = [self.local_store.get(key) for key in keys]
        missing = [i for i, v in enumerate(ret) if v is None]
        for i, value in zip(missing, self.remote_store.batched_get([keys[i] for i in missing])):
            if value is not None:
                self.local_store.put(keys[i], value)
                ret[i] = value
        return ret

    def close(self):
        self.local_store.close()
        self.remote_store.close()
