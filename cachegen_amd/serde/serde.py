"""Serializer / Deserializer plug-in interface
(LMCache/lmcache/storage_backend/serde/serde.py:9-63 in the reference)."""
import abc
import logging
import time

import torch

logger = logging.getLogger("cachegen_amd")


class Serializer(metaclass=abc.ABCMeta):
    @abc.abstractmethod
    def to_bytes(self, t: torch.Tensor) -> bytes:
        """Serialize a tensor (data and metadata) to bytes."""
        raise NotImplementedError


class Deserializer(metaclass=abc.ABCMeta):
    @abc.abstractmethod
    def from_bytes(self, bs: bytes) -> torch.Tensor:
        """Rebuild the tensor from `to_bytes` output."""
        raise NotImplementedError


class SerializerDebugWrapper(Serializer):
    def __init__(self, s: Serializer):
        self.s = s

    def to_bytes(self, t: torch.Tensor) -> bytes:
        start = time.perf_counter()
        bs = self.s.to_bytes(t)
        logger.debug("Serialization took %.2f seconds", time.perf_counter() - start)
        return bs

    def __getattr__(self, name):           # whatever else the wrapped serializer offers
        return getattr(self.s, name)


class DeserializerDebugWrapper(Deserializer):
    def __init__(self, d: Deserializer):
        self.d = d

    def from_bytes(self, bs: bytes) -> torch.Tensor:
        start = time.perf_counter()
        ret = self.d.from_bytes(bs)
        logger.debug("Deserialization took %.2f ms", (time.perf_counter() - start) * 1000)
        return ret

    def __getattr__(self, name):
        return getattr(self.d, name)
