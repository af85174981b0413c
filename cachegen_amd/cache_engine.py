"""The chunked KV-cache store in front of the codec
(LMCache/lmcache/cache_engine.py:22-371 in the reference).

`store` cuts a context's KV cache into chunks of `chunk_size` tokens keyed by the SHA-256 of
the token prefix up to and including the chunk, `retrive` returns the KV cache of the longest
stored prefix of a token sequence.  Keys and hashes are the reference's, so stores written by
either implementation are found by the other.  Unlike the reference, the cache is stacked
into one tensor once and handed to the backend whole, so that a compressing backend encodes
all chunks in one pass and decodes them in place instead of chunk by chunk with a
concatenation at the end."""
import hashlib
import logging
import time
from typing import Iterator, List, Optional, Tuple

import torch

from .config import LMCacheEngineConfig, LMCacheEngineMetadata
from .storage_backend import CreateStorageBackend
from .utils import CacheEngineKey, KVCache

logger = logging.getLogger("cachegen_amd")


def _token_dim(fmt: str) -> int:
    """Token dimension of one layer's key or value tensor."""
    if fmt == "huggingface":
        return 1
    if fmt == "vllm":
        return 0
    raise ValueError(f"Invalid format: {fmt}")


class LMCacheEngine:
    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
        self.config = config
        self.metadata = metadata
        self.chunk_size = config.chunk_size
        # where chunks are staged before they go to the store: the GPU unless the local store is
        # on the CPU (cache_engine.py:37-41), or there is no GPU and no local store at all
        no_gpu_remote = config.local_device is None and not torch.cuda.is_available()
        self.device = "cpu" if config.local_device == "cpu" or no_gpu_remote else "cuda"
        self.engine_ = CreateStorageBackend(config, metadata)

    # ---- keys ------------------------------------------------------------------------------
    def _make_key(self, chunk_hash: str, fmt: str) -> CacheEngineKey:
        return CacheEngineKey(fmt, self.metadata.model_name, self.metadata.world_size,
                              self.metadata.worker_id, chunk_hash)

    def _hash(self, tokens: torch.Tensor, prefix_hash: str) -> str:
        """cache_engine.py:68-74: the chunk's token ids as raw bytes of their own dtype."""
        return hashlib.sha256(prefix_hash.encode("ascii") + tokens.cpu().numpy().tobytes()).hexdigest()

    def _prefix_hashes(self, tokens: torch.Tensor) -> Iterator[str]:
        prefix_hash = ""
        host = tokens.cpu()                     # one copy, not one per chunk
        for i in range(0, len(host), self.chunk_size):
            prefix_hash = self._hash(host[i:i + self.chunk_size], prefix_hash)
            yield prefix_hash

    def _num_tokens_in_kv(self, kv_tensors: KVCache, fmt: str) -> int:
        return kv_tensors[0][0].shape[_token_dim(fmt)]

    # ---- layout ----------------------------------------------------------------------------
    @staticmethod
    def _tuple_kv_to_blob(kv_tensors: KVCache) -> torch.Tensor:
        """Nested tuple -> one tensor with two leading dimensions (layer, key|value)."""
        return torch.stack([torch.stack(pair, dim=0) for pair in kv_tensors], dim=0)

    @staticmethod
    def _blob_to_tuple_kv(blob: torch.Tensor) -> KVCache:
        return tuple((layer[0], layer[1]) for layer in torch.unbind(blob, dim=0))

    # ---- store -----------------------------------------------------------------------------
    def store(self, tokens: torch.Tensor, kv_tensors: KVCache, skip_existing: bool = True,
              blocking: bool = True) -> None:
        """tokens: [seq_len]; kv_tensors: per layer (key, value), each [num_tokens, num_heads,
        head_size] (vllm) or [num_heads, num_tokens, head_size] (huggingface), no batch
        dimension.  Chunks already present are left alone unless skip_existing is False."""
        start = time.perf_counter()
        fmt = self.metadata.fmt
        assert len(tokens.shape) == 1, f"Invalid shape of tokens: {tokens.shape}"
        assert len(kv_tensors) > 0, "Empty kv_tensors"
        assert len(tokens) == self._num_tokens_in_kv(kv_tensors, fmt), \
            "Number of tokens in the kv cache does not match the input tokens"

        keys: List[Optional[CacheEngineKey]] = []
        for chunk_hash in self._prefix_hashes(tokens):
            key = self._make_key(chunk_hash, fmt)
            keys.append(None if skip_existing and self.engine_.contains(key) else key)
        n_chunks = 0
        if any(key is not None for key in keys):
            blob = self._tuple_kv_to_blob(kv_tensors).to(self.device)
            n_chunks = self.engine_.put_chunks(keys, blob, self.chunk_size, fmt, blocking=blocking)
        logger.info("Stored/updated %d chunks, total time %.2fs", n_chunks, time.perf_counter() - start)

    # ---- retrieve --------------------------------------------------------------------------
    def retrive(self, tokens: torch.Tensor, device: str = "cuda") -> Tuple[KVCache, int]:
        """The KV cache of the longest stored prefix of `tokens` (whole chunks) as a nested
        tuple on `device`, and its number of tokens; ((), 0) if the first chunk is missing."""
        start = time.perf_counter()
        fmt = self.metadata.fmt
        tdim = _token_dim(fmt)
        keys = (self._make_key(chunk_hash, fmt) for chunk_hash in self._prefix_hashes(tokens))

        if hasattr(self.engine_, "get_chunks_concat"):
            blob = self.engine_.get_chunks_concat(keys, fmt)
        else:
            chunks = []
            for chunk in self.engine_.batched_get(keys):
                if chunk is None:
                    break
                chunks.append(chunk)
            blob = torch.cat(chunks, dim=tdim + 2) if chunks else None
        if blob is None:
            logger.info("Retrived 0 chunks")
            return (), 0
        ret = self._blob_to_tuple_kv(blob.to(device))
        ntokens = ret[0][0].shape[tdim]
        logger.info("Retrived %d tokens -- elapsed time %.4f", ntokens, time.perf_counter() - start)
        return ret, ntokens

    def persist(self):
        """Kept for callers of the reference's interface; stores here have nothing to flush to."""
        if hasattr(self.engine_, "persist"):
            self.engine_.persist()

    def close(self):
        self.engine_.close()


class LMCacheEngineBuilder:
    """One engine per instance id (cache_engine.py:332-371)."""
    _instances = {}
    _cfgs = {}
    _metadatas = {}

    @classmethod
    def get_or_create(cls, instance_id: str, config: LMCacheEngineConfig,
                      metadata: LMCacheEngineMetadata) -> LMCacheEngine:
        if instance_id not in cls._instances:
            cls._instances[instance_id] = LMCacheEngine(config, metadata)
            cls._cfgs[instance_id] = config
            cls._metadatas[instance_id] = metadata
            return cls._instances[instance_id]
        if cls._cfgs[instance_id] != config or cls._metadatas[instance_id] != metadata:
            raise ValueError(f"Instance {instance_id} already exists with a different configuration or metadata.")
        return cls._instances[instance_id]

    @classmethod
    def get(cls, instance_id: str) -> Optional[LMCacheEngine]:
        return cls._instances.get(instance_id)
