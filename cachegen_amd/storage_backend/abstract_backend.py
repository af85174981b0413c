"""Interface of a chunk store (LMCache/lmcache/storage_backend/abstract_backend.py:11-112)."""
import abc
from typing import Iterable, Iterator, List, Optional, Tuple

import torch

from ..utils import CacheEngineKey


class LMCBackendInterface(metaclass=abc.ABCMeta):
    @abc.abstractmethod
    def put(self, key: CacheEngineKey, kv_chunk: torch.Tensor, blocking: bool = True) -> None:
        """Store one chunk: a tensor [L, 2, ...] without a batch dimension."""
        raise NotImplementedError

    @abc.abstractmethod
    def contains(self, key: CacheEngineKey) -> bool:
        raise NotImplementedError

    @abc.abstractmethod
    def get(self, key: CacheEngineKey) -> Optional[torch.Tensor]:
        """The chunk stored under `key`, or None."""
        raise NotImplementedError

    def batched_put(self, keys_and_chunks: Iterable[Tuple[CacheEngineKey, torch.Tensor]],
                    blocking: bool = True) -> int:
        """Stores every (key, chunk); returns how many."""
        n = 0
        for key, chunk in keys_and_chunks:
            self.put(key, chunk, blocking=blocking)
            n += 1
        return n

    def batched_get(self, keys: Iterable[CacheEngineKey]) -> Iterator[Optional[torch.Tensor]]:
        for key in keys:
            yield self.get(key) if self.contains(key) else None

    # --- whole-tensor forms (not in the reference) -------------------------------------
    def put_chunks(self, keys: List[Optional[CacheEngineKey]], blob: torch.Tensor, chunk_size: int,
                   fmt: str, blocking: bool = True) -> int:
        """Stores chunk i of `blob` ([L,2,T,H,D] for fmt "vllm", [L,2,H,T,D] for "huggingface",
        cut every `chunk_size` tokens) under keys[i]; chunks whose key is None are skipped.
        Backends that encode override this to encode all chunks in one pass."""
        tdim = 2 if fmt == "vllm" else 3
        T = blob.shape[tdim]
        n = 0
        for i, key in enumerate(keys):
            if key is None:
                continue
            t0 = i * chunk_size
            self.put(key, blob.narrow(tdim, t0, min(chunk_size, T - t0)), blocking=blocking)
            n += 1
        return n

    def close(self) -> None:
        pass
