"""Key and type definitions shared by the cache engine and its backends
(LMCache/lmcache/utils.py:8-31 in the reference)."""
from dataclasses import dataclass
from typing import Tuple

import torch

# one (key, value) pair per layer, each [num_tokens, num_heads, head_size] ("vllm") or
# [num_heads, num_tokens, head_size] ("huggingface"): no batch dimension
KVCache = Tuple[Tuple[torch.Tensor, torch.Tensor], ...]


@dataclass(frozen=True)
class CacheEngineKey:
    fmt: str
    model_name: str
    world_size: int
    worker_id: int
    chunk_hash: str

    def to_string(self) -> str:
        return f"{self.fmt}@{self.model_name}@{self.world_size}@{self.worker_id}@{self.chunk_hash}"

    @staticmethod
    def from_string(s: str) -> "CacheEngineKey":
        parts = s.split("@")
        if len(parts) != 5:
            raise ValueError(f"Invalid key string: {s}")
        return CacheEngineKey(parts[0], parts[1], int(parts[2]), int(parts[3]), parts[4])
