"""The configuration records of the cache engine and its serializers
(LMCache/lmcache/config.py:6-87 in the reference)."""
import re
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

    @staticmethod
    def from_legacy(chunk_size=256, backend="cuda", persist_path=None, remote_serde="torch",
                    pipelined_backend=False):
        """`backend` is "cpu", "cuda" (local only) or a URL scheme://host:port (remote only);
        `persist_path` is accepted and ignored, as in the reference (config.py:37-55)."""
        if backend in ("cpu", "cuda"):
            local_device, remote_url = backend, None
        elif re.match(r"(.*)://(.*):(\d+)", backend):
            local_device, remote_url = None, backend
        else:
            raise ValueError(f"Invalid backend: {backend}")
        return LMCacheEngineConfig(chunk_size, local_device, remote_url, remote_serde, pipelined_backend)

    @staticmethod
    def from_file(file_path):
        """Keys of the YAML file: chunk_size, local_device, remote_url, remote_serde,
        pipelined_backend (config.py:57-73)."""
        import yaml
        with open(file_path, "r") as fin:
            config = yaml.safe_load(fin) or {}
        return LMCacheEngineConfig(config.get("chunk_size", 256), config.get("local_device", None),
                                   config.get("remote_url", None), config.get("remote_serde", "torch"),
                                   config.get("pipelined_backend", False))


class GlobalConfig:
    enable_debug: bool = True

    @classmethod
    def set_debug(cls, enable):
        cls.enable_debug = enable

    @classmethod
    def is_debug(cls):
        return cls.enable_debug
