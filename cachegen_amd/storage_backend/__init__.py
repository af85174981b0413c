"""Chunk stores of the cache engine (LMCache/lmcache/storage_backend/__init__.py:11-31)."""
from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from .abstract_backend import LMCBackendInterface
from .hybrid_backend import LMCHybridBackend
from .local_backend import LMCLocalBackend
from .remote_backend import LMCPipelinedRemoteBackend, LMCRemoteBackend


def CreateStorageBackend(config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata) -> LMCBackendInterface:
    """local_device only: local store; remote_url only: remote store; both: hybrid."""
    local, remote = config.local_device, config.remote_url
    if local is None and isinstance(remote, str):
        return LMCRemoteBackend(config, metadata)
    if isinstance(local, str) and remote is None:
        return LMCLocalBackend(config)
    if isinstance(local, str) and isinstance(remote, str):
        return LMCHybridBackend(config, metadata)
    raise ValueError(f"Invalid configuration: {config}")


__all__ = ["LMCBackendInterface", "LMCLocalBackend", "LMCRemoteBackend", "LMCPipelinedRemoteBackend",
           "LMCHybridBackend", "CreateStorageBackend"]
