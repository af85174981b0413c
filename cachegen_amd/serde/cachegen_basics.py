"""Per-model quantization tables and the wire containers of the codec
(LMCache/lmcache/storage_backend/serde/cachegen_basics.py in the reference).

Field names, table values and the QUANT_LEVEL environment switch are the
reference's (cachegen_basics.py:10-96, 124-156), so objects and pickles carry the
same fields."""
import io
import os
import pickle
from dataclasses import dataclass
from typing import List

import torch

CACHEGEN_GPU_MAX_TOKENS_PER_CHUNK = 256


@dataclass
class CacheGenConfig:
    key_first_layers: int
    key_second_layers: int
    key_third_layers: int
    key_first_bins: int
    key_second_bins: int
    key_third_bins: int
    value_first_layers: int
    value_first_bins: int
    value_second_bins: int

    def __getitem__(self, key: str) -> int:
        return getattr(self, key)

    @staticmethod
    def _tiers(num_layers, first, second, k_bins, v_first, v_bins):
        return CacheGenConfig(
            key_first_layers=first, key_second_layers=second, key_third_layers=num_layers,
            key_first_bins=k_bins[0], key_second_bins=k_bins[1], key_third_bins=k_bins[2],
            value_first_layers=v_first, value_first_bins=v_bins[0], value_second_bins=v_bins[1])

    @staticmethod
    def from_model_name(model_name: str) -> "CacheGenConfig":
        """Names containing "Mistral-7B" read the QUANT_LEVEL environment variable
        ("1", "2" or "3"; KeyError if unset, None for any other value); the listed 7B
        names use the level-2 table and the 70B name its own (cachegen_basics.py:27-96)."""
        family_7b = ["mistralai/Mistral-7B-Instruct-v0.2", "mistral-community/Mistral-7B-v0.2",
                     "lmsys/longchat-7b-16k"]
        family_70b = ["Yukang/LongAlpaca-70B-16k"]
        levels_7b = {
            "1": ((16, 16, 12), (16, 12)),
            "2": ((32, 16, 16), (32, 16)),
            "3": ((32, 32, 32), (32, 32)),
        }
        if "Mistral-7B" in model_name:
            level = os.environ["QUANT_LEVEL"]
            if level in levels_7b:
                k, v = levels_7b[level]
                return CacheGenConfig._tiers(32, 10, 20, k, 2, v)
            return None
        elif model_name in family_7b:
            k, v = levels_7b["2"]
            return CacheGenConfig._tiers(32, 10, 20, k, 2, v)
        elif model_name in family_70b:
            return CacheGenConfig._tiers(80, 20, 40, (32, 32, 16), 20, (32, 16))
        else:
            raise ValueError(f"Model {model_name} is not supported")

    @staticmethod
    def from_layer_tiers(num_layers, key_tiers, value_tiers) -> "CacheGenConfig":
        """Explicit table: key_tiers = [(first_layers, bins), (second_layers, bins), bins_rest],
        value_tiers = [(first_layers, bins), bins_rest]."""
        (k1, kb1), (k2, kb2), kb3 = key_tiers
        (v1, vb1), vb2 = value_tiers
        return CacheGenConfig._tiers(num_layers, k1, k2, (kb1, kb2, kb3), v1, (vb1, vb2))


def make_key_bins(config: CacheGenConfig) -> torch.Tensor:
    """float32 [key_third_layers] on the CPU (cachegen_encoder.py:311-316)."""
    ret = torch.zeros(config.key_third_layers)
    ret.fill_(config.key_third_bins)
    ret[:config.key_second_layers] = config.key_second_bins
    ret[:config.key_first_layers] = config.key_first_bins
    return ret


def make_value_bins(config: CacheGenConfig) -> torch.Tensor:
    """float32 [key_third_layers] on the CPU (cachegen_encoder.py:318-322)."""
    ret = torch.zeros(config.key_third_layers)
    ret.fill_(config.value_second_bins)
    ret[:config.value_first_layers] = config.value_first_bins
    return ret


@dataclass
class CacheGenGPUBytestream:
    bytestream: torch.Tensor          # uint8 [n]: streams in (layer, channel) order
    bytestream_lengths: torch.Tensor  # int32 [2L, C]
    ntokens: int

    def __getitem__(self, key: str):
        return getattr(self, key)


@dataclass
class CacheGenGPUEncoderOutput:
    data_chunks: List[CacheGenGPUBytestream]
    cdf: torch.Tensor                 # int16 [2L, C, Lp]
    max_tensors_key: torch.Tensor     # input dtype [L, T, 1]
    max_tensors_value: torch.Tensor
    num_heads: int
    head_size: int

    def __getitem__(self, key: str):
        return getattr(self, key)

    def to_bytes(self) -> bytes:
        with io.BytesIO() as f:
            pickle.dump(self, f)
            return f.getvalue()

    @staticmethod
    def from_bytes(bs: bytes) -> "CacheGenGPUEncoderOutput":
        """Reads a container written here or by the reference (cachegen_basics.py:146-156 pickles
        the same two dataclasses under `lmcache.storage_backend.serde.cachegen_basics`).  Only the
        globals such a pickle needs are resolved; anything else a blob names is refused, so a
        store cannot make this call run code of its choosing."""
        with io.BytesIO(bs) as f:
            return _ContainerUnpickler(f).load()


def _load_storage(b: bytes):
    # what torch.storage._load_from_bytes does, without its general unpickling
    return torch.load(io.BytesIO(b), weights_only=True)


class _ContainerUnpickler(pickle.Unpickler):
    """Unpickler for CacheGenGPUEncoderOutput blobs: the two container classes under this
    package's module path and under the reference's, and the three helpers with which torch
    pickles a tensor (the storage's bytes are read with `weights_only=True`)."""

    _CONTAINER_MODULES = ("cachegen_amd.serde.cachegen_basics", "lmcache.storage_backend.serde.cachegen_basics")
    _CONTAINER_CLASSES = ("CacheGenGPUEncoderOutput", "CacheGenGPUBytestream", "CacheGenEncoderOutput")

    def find_class(self, module, name):
        if module in self._CONTAINER_MODULES and name in self._CONTAINER_CLASSES:
            return globals()[name]
        if (module, name) == ("torch._utils", "_rebuild_tensor_v2"):
            return torch._utils._rebuild_tensor_v2
        if (module, name) == ("torch.storage", "_load_from_bytes"):
            return _load_storage
        if (module, name) == ("collections", "OrderedDict"):
            import collections
            return collections.OrderedDict
        raise pickle.UnpicklingError("CacheGen container: refusing to load %s.%s" % (module, name))


# The reference's tests load the encoder output under this older name as well
# (LMCache/tests/test_serde.py:6,43); unpickling does not depend on it.
CacheGenEncoderOutput = CacheGenGPUEncoderOutput
