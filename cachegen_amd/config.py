"""The two configuration records the serializer constructors take
(LMCache/lmcache/config.py:6-87 in the reference), reduced to what the codec reads."""
from dataclasses import dataclass
from typing import Optional


@dataclass
class LMCacheEngineMetadata:
    model_name: str      # selects the per-layer bins table
    world_size: int
    worker_id: int
    fmt: str             # "vllm" or "huggingface": layout of the KV tensors


@dataclass
class LMCacheEngineConfig:
    chunk_size: int
    local_device: Optional[str]
    remote_url: Optional[str]
    remote_serde: Optional[str]
    pipelined_backend: bool

    @staticmethod
    def from_defaults(chunk_size=256, local_device="cuda", remote_url="redis://localhost:6379",
                      remote_serde="torch", pipelined_backend=False):
        return LMCacheEngineConfig(chunk_size, local_device, remote_url, remote_serde, pipelined_backend)


class GlobalConfig:
    enable_debug: bool = True

    @classmethod
    def set_debug(cls, enable):
        cls.enable_debug = enable

    @classmethod
    def is_debug(cls):
        return cls.enable_debug
