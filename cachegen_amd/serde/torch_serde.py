"""Uncompressed serde: torch.save / torch.load of the chunk tensor
(LMCache/lmcache/storage_backend/serde/torch_serde.py:10-62).  Loading is restricted to
tensor data (`weights_only=True`), which is all a chunk holds."""
import io

import torch

from .serde import Deserializer, Serializer


class TorchSerializer(Serializer):
    def to_bytes(self, t: torch.Tensor) -> bytes:
        with io.BytesIO() as f:
            torch.save(t, f)
            return f.getvalue()


class TorchDeserializer(Deserializer):
    def from_bytes(self, b: bytes) -> torch.Tensor:
        with io.BytesIO(b) as f:
            return torch.load(f, weights_only=True)
