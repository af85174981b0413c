"""Serde plug-ins (LMCache/lmcache/storage_backend/serde/__init__.py:7-18 in the reference).
"torch" stores the tensor as it is, "cachegen" compresses it, and "cachegen-flat" (not in the
reference) is the same codec writing the flat container of `wire` instead of a pickle."""
from ..config import GlobalConfig, LMCacheEngineConfig, LMCacheEngineMetadata
from .cachegen_decoder import CacheGenDeserializer
from .cachegen_encoder import CacheGenSerializer
from .serde import Deserializer, DeserializerDebugWrapper, Serializer, SerializerDebugWrapper
from .torch_serde import TorchDeserializer, TorchSerializer


def CreateSerde(serde_type: str, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
    if serde_type == "torch":
        s, d = TorchSerializer(), TorchDeserializer()
    elif serde_type == "cachegen":
        s, d = CacheGenSerializer(config, metadata), CacheGenDeserializer(config, metadata)
    elif serde_type == "cachegen-flat":      # not in the reference: same codec, flat container
        s, d = CacheGenSerializer(config, metadata, wire_format="flat"), CacheGenDeserializer(config, metadata)
    else:
        raise ValueError(f"Invalid serde type: {serde_type}")
    if GlobalConfig.is_debug():
        return SerializerDebugWrapper(s), DeserializerDebugWrapper(d)
    return s, d


__all__ = ["Serializer", "Deserializer", "TorchSerializer", "TorchDeserializer", "CacheGenDeserializer",
           "CacheGenSerializer", "CreateSerde"]
