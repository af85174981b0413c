"""Key and type definitions shared by the cache engine and its stores
(LMCache/lmcache/utils.py:8-31 in the reference)."""
from typing import NamedTuple, Tuple

import torch

# one (key, value) pair per layer, each [num_tokens, num_heads, head_size] ("vllm") or
# [num_heads, num_tokens, head_size] ("huggingface"): no batch dimension
KVCache = Tuple[Tuple[torch.Tensor, torch.Tensor], ...]


class CacheEngineKey(NamedTuple):
    """What a stored chunk is filed under.  Its string form, the five fields joined by "@",
    is the key on the remote side, so a model name must not contain "@"."""
    fmt: str
    model_name: str
    world_size: int
    worker_id: int
    chunk_hash: str

    def to_string(self) -> str:
        return "@".join(str(field) for field in self)

    @classmethod
    def from_string(cls, s: str) -> "CacheEngineKey":
        fields = s.split("@")
        if len(fields) != 5:
            raise ValueError(f"Invalid key string: {s}")
        fmt, model_name, world_size, worker_id, chunk_hash = fields
        return cls(fmt, model_name, int(world_size), int(worker_id), chunk_hash)
