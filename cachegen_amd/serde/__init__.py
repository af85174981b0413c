"""Serde plug-ins (LMCache/lmcache/storage_backend/serde/__init__.py:7-18 in the reference).
Only the "cachegen" serde is provided here, with "cachegen-flat" as its variant that writes the
flat container of `wire` instead of a pickle."""
from ..config import GlobalConfig, LMCacheEngineConfig, LMCacheEngineMetadata
from .cachegen_decoder import CacheGenDeserializer
from .cachegen_encoder import CacheGenSerializer
from .serde import Deserializer, DeserializerDebugWrapper, Serializer, SerializerDebugWrapper


def CreateSerde(serde_type: str, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
    if serde_type == "cachegen":
        s, d = CacheGenSerializer(config, metadata), CacheGenDeserializer(config, metadata)
    elif serde_type == "cachegen-flat":      # not in the reference: same codec, flat container
        s, d = CacheGenSerializer(config, metadata, wire_format="flat"), CacheGenDeserializer(config, metadata)
    else:
        raise ValueError(f"Invalid serde type: {serde_type}")
    if GlobalConfig.is_debug():
        return SerializerDebugWrapper(s), DeserializerDebugWrapper(d)
    return s, d


__all__ = ["Serializer", "Deserializer", "CacheGenDeserializer", "CacheGenSerializer", "CreateSerde"]
