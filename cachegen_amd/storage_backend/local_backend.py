"""Chunk store in local CPU or GPU memory
(LMCache/lmcache/storage_backend/local_backend.py:15-86)."""
import logging
from typing import Optional

import torch

from ..config import LMCacheEngineConfig
from ..utils import CacheEngineKey
from .abstract_backend import LMCBackendInterface

logger = logging.getLogger("cachegen_amd")


class LMCLocalBackend(LMCBackendInterface):
    def __init__(self, config: LMCacheEngineConfig):
        self.chunk_size = config.chunk_size
        self.config = config
        self.dict = {}

    def contains(self, key: CacheEngineKey) -> bool:
        return key in self.dict

    def put(self, key: CacheEngineKey, kv_chunk: torch.Tensor, blocking: bool = True) -> None:
        if not blocking:
            logger.warning("Non-blocking is not implemented for local backend")
        self.dict[key] = kv_chunk

    def get(self, key: CacheEngineKey) -> Optional[torch.Tensor]:
        return self.dict.get(key, None)

    def put_chunks(self, keys, blob, chunk_size, fmt, blocking=True) -> int:
        """Every stored chunk is a copy of its own, so the cache never aliases the caller's
        tensor."""
        tdim = 2 if fmt == "vllm" else 3
        T = blob.shape[tdim]
        n = 0
        for i, key in enumerate(keys):
            if key is None:
                continue
            t0 = i * chunk_size
            self.dict[key] = blob.narrow(tdim, t0, min(chunk_size, T - t0)).clone(memory_format=torch.contiguous_format)
            n += 1
        return n
