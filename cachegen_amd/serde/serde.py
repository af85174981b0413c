"""Serializer / Deserializer plug-in interface
(LMCache/lmcache/storage_backend/serde/serde.py:9-63 in the reference): a serializer turns a
chunk tensor into bytes, a deserializer turns them back."""
import abc
import logging
import time

import torch

logger = logging.getLogger("cachegen_amd")


class Serializer(metaclass=abc.ABCMeta):
    @abc.abstractmethod
    def to_bytes(self, t: torch.Tensor) -> bytes:
        """The tensor, data and whatever is needed to rebuild it, as bytes."""
        raise NotImplementedError


class Deserializer(metaclass=abc.ABCMeta):
    @abc.abstractmethod
    def from_bytes(self, bs: bytes) -> torch.Tensor:
        """The tensor that `to_bytes` was given (or its lossy reconstruction)."""
        raise NotImplementedError


class _Timed:
    """Wraps a serde object: the one interface call is timed into the debug log, everything
    else the wrapped object offers passes through."""

    def __init__(self, inner, what):
        self._inner = inner
        self._what = what

    def _run(self, fn, arg):
        t0 = time.perf_counter()
        ret = fn(arg)
        logger.debug("%s took %.2f ms", self._what, (time.perf_counter() - t0) * 1e3)
        return ret

    def __getattr__(self, name):
        return getattr(self._inner, name)


class SerializerDebugWrapper(_Timed, Serializer):
    def __init__(self, s: Serializer):
        _Timed.__init__(self, s, "Serialization")

    @property
    def s(self) -> Serializer:          # the wrapped serializer, under the reference's attribute name
        return self._inner

    def to_bytes(self, t: torch.Tensor) -> bytes:
        return self._run(self._inner.to_bytes, t)


class DeserializerDebugWrapper(_Timed, Deserializer):
    def __init__(self, d: Deserializer):
        _Timed.__init__(self, d, "Deserialization")

    @property
    def d(self) -> Deserializer:
        return self._inner

    def from_bytes(self, bs: bytes) -> torch.Tensor:
        return self._run(self._inner.from_bytes, bs)
