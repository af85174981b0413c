"""Chunk store behind a connector, with serialized chunks
(LMCache/lmcache/storage_backend/remote_backend.py:19-283).

With a CacheGen serde the whole-tensor forms do what the codec is built for: `put_chunks`
encodes every chunk of a KV cache in one pass over the tensor, and `get_chunks_concat` decodes
every chunk it finds straight into its token range of one output tensor."""
import logging
import queue
import threading
from typing import Iterable, List, Optional

import torch

from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from ..serde import CreateSerde
from ..utils import CacheEngineKey
from .abstract_backend import LMCBackendInterface
from .connector import CreateConnector

logger = logging.getLogger("cachegen_amd")


class LMCRemoteBackend(LMCBackendInterface):
    class _EndSignal:
        pass

    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
        self.existing_keys = set()
        self.connection = CreateConnector(config.remote_url)
        self.serializer, self.deserializer = CreateSerde(config.remote_serde, config, metadata)
        self.put_queue = queue.Queue()          # (key, chunk) or (key, None, blob bytes) for the worker
        self.put_thread = threading.Thread(target=self.put_worker, daemon=True)
        self.put_thread.start()

    # ---- keys --------------------------------------------------------------------------
    def _combine_key(self, key: CacheEngineKey) -> str:
        return key.to_string()

    def _split_key(self, key: str) -> CacheEngineKey:
        return CacheEngineKey.from_string(key)

    def list(self) -> List[CacheEngineKey]:
        """Keys on the remote side; also refreshes the local record of them."""
        keys = [self._split_key(k) for k in self.connection.list()]
        self.existing_keys.update(keys)
        return keys

    def contains(self, key: CacheEngineKey) -> bool:
        if key in self.existing_keys:
            return True
        found = bool(self.connection.exists(self._combine_key(key)))
        if found:
            self.existing_keys.add(key)
        return found

    # ---- put ---------------------------------------------------------------------------
    def put_worker(self):
        while True:
            item = self.put_queue.get()
            try:
                if isinstance(item, LMCRemoteBackend._EndSignal):
                    return
                key, chunk, blob = item
                if blob is None:
                    if chunk.is_cuda:
                        with torch.cuda.stream(torch.cuda.Stream(device=chunk.device)):
                            blob = self.serializer.to_bytes(chunk)
                    else:
                        blob = self.serializer.to_bytes(chunk)
                self._send(key, blob)
            except Exception:                   # keep the worker alive: a lost put is a cache miss later
                logger.exception("asynchronous put failed")
            finally:
                self.put_queue.task_done()

    def _send(self, key: CacheEngineKey, blob: bytes) -> None:
        self.connection.set(self._combine_key(key), blob)
        self.existing_keys.add(key)

    def put_blocking(self, key: CacheEngineKey, kv_chunk: torch.Tensor) -> None:
        self._send(key, self.serializer.to_bytes(kv_chunk))

    def put(self, key: CacheEngineKey, kv_chunk: torch.Tensor, blocking: bool = True) -> None:
        if blocking:
            self.put_blocking(key, kv_chunk)
        else:
            self.put_queue.put((key, kv_chunk.clone(), None))

    def put_chunks(self, keys, blob, chunk_size, fmt, blocking=True) -> int:
        wanted = [i for i, key in enumerate(keys) if key is not None]
        if not wanted:
            return 0
        if not hasattr(self.serializer, "to_bytes_chunks"):
            return super().put_chunks(keys, blob, chunk_size, fmt, blocking)
        # one pass of the codec over the token range that holds every wanted chunk
        tdim = 2 if fmt == "vllm" else 3
        first, last = wanted[0], wanted[-1]
        t0 = first * chunk_size
        t1 = min((last + 1) * chunk_size, blob.shape[tdim])
        blobs = self.serializer.to_bytes_chunks(blob.narrow(tdim, t0, t1 - t0), chunk_size)
        for i in wanted:
            if blocking:
                self._send(keys[i], blobs[i - first])
            else:
                self.put_queue.put((keys[i], None, blobs[i - first]))
        return len(wanted)

    # ---- get ---------------------------------------------------------------------------
    def get_bytes(self, key: CacheEngineKey) -> Optional[bytes]:
        if not self.contains(key):
            return None
        bs = self.connection.get(self._combine_key(key))
        return bs if bs else None

    def get(self, key: CacheEngineKey) -> Optional[torch.Tensor]:
        bs = self.get_bytes(key)
        return None if bs is None else self.deserializer.from_bytes(bs)

    def get_chunks_concat(self, keys: Iterable[CacheEngineKey], fmt: str) -> Optional[torch.Tensor]:
        """The chunks stored under the leading keys that are present, side by side along the
        token dimension in one tensor, or None if the first key is missing.  Chunks in the flat
        container are decoded in place; anything else is decoded and copied."""
        blobs = []
        for key in keys:
            bs = self.get_bytes(key)
            if bs is None:
                break
            blobs.append(bs)
        if not blobs:
            return None
        tdim = 2 if fmt == "vllm" else 3
        shapes = [self.deserializer.chunk_shape(bs) if hasattr(self.deserializer, "chunk_shape") else None
                  for bs in blobs]
        if any(s is None for s in shapes):
            return torch.cat([self.deserializer.from_bytes(bs) for bs in blobs], dim=tdim)
        shape = list(shapes[0])
        shape[tdim] = sum(s[tdim] for s in shapes)
        out = torch.empty(shape, dtype=torch.bfloat16 if fmt == "vllm" else torch.float16, device="cuda")
        t0 = 0
        for bs, s in zip(blobs, shapes):
            self.deserializer.from_bytes_into(bs, out.narrow(tdim, t0, s[tdim]))
            t0 += s[tdim]
        return out

    # ---- shutdown ----------------------------------------------------------------------
    def flush(self) -> None:
        """Waits until every asynchronous put has been sent."""
        self.put_queue.join()

    def close(self):
        if self.put_thread is not None and self.put_thread.is_alive():
            self.put_queue.put(self._EndSignal())
            self.put_thread.join()
        self.put_thread = None


class LMCPipelinedRemoteBackend(LMCRemoteBackend):
    """`batched_get` overlaps fetching chunk i+1 with deserializing chunk i: one thread pulls
    bytes from the connector, one decodes them (remote_backend.py:180-283).  Results keep the
    order of the keys and stop at the first missing one."""

    def batched_get(self, keys: Iterable[CacheEngineKey]):
        fetched: "queue.Queue" = queue.Queue(maxsize=4)
        done = object()

        def fetch():
            try:
                for key in keys:
                    bs = self.get_bytes(key)
                    fetched.put(bs)
                    if bs is None:
                        break
            finally:
                fetched.put(done)

        worker = threading.Thread(target=fetch, daemon=True)
        worker.start()
        results = []
        missing = False
        while True:
            item = fetched.get()
            if item is done:
                break
            if item is None or missing:
                missing = True
                results.append(None)
                continue
            results.append(self.deserializer.from_bytes(item))
        worker.join()
        return results
