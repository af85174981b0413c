"""Serde plug-ins (LMCache/lmcache/storage_backend/serde/__init__.py:7-18 in the reference).

  "torch"          the chunk tensor as torch.save writes it
  "cachegen"       the codec, in the reference's pickle container
  "cachegen-flat"  the same codec in the flat container of `wire` (not in the reference)
  "cachegen-compact"  the same in version 2 of that container (tables as histogram counts)
"""
from ..config import GlobalConfig, LMCacheEngineConfig, LMCacheEngineMetadata
from .cachegen_decoder import CacheGenDeserializer
from .cachegen_encoder import CacheGenSerializer
from .serde import Deserializer, DeserializerDebugWrapper, Serializer, SerializerDebugWrapper
from .torch_serde import TorchDeserializer, TorchSerializer

_FACTORIES = {
    "torch": lambda config, metadata: (TorchSerializer(), TorchDeserializer()),
    "cachegen": lambda config, metadata: (CacheGenSerializer(config, metadata),
                                          CacheGenDeserializer(config, metadata)),
    "cachegen-flat": lambda config, metadata: (CacheGenSerializer(config, metadata, wire_format="flat"),
                                               CacheGenDeserializer(config, metadata)),
    "cachegen-compact": lambda config, metadata: (CacheGenSerializer(config, metadata, wire_format="compact"),
                                                  CacheGenDeserializer(config, metadata)),
}


def CreateSerde(serde_type: str, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
    """(serializer, deserializer) of the named kind, timed into the debug log when
    GlobalConfig.is_debug()."""
    try:
        make = _FACTORIES[serde_type]
    except KeyError:
        raise ValueError(f"Invalid serde type: {serde_type}") from None
    s, d = make(config, metadata)
    if GlobalConfig.is_debug():
        s, d = SerializerDebugWrapper(s), DeserializerDebugWrapper(d)
    return s, d


__all__ = ["Serializer", "Deserializer", "TorchSerializer", "TorchDeserializer", "CacheGenDeserializer",
           "CacheGenSerializer", "CreateSerde"]
