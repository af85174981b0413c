"""The cache engine and its stores (cachegen_amd/cache_engine.py, storage_backend/): the
behaviours the reference's own tests check (LMCache/tests/test_cache_engine.py,
test_backends.py, test_connector.py), run against the local store and an in-process remote
store on the CPU, and on the GPU against the compressing serdes, where a retrieved chunk must
equal the serializer's own round trip of that chunk bit for bit."""
import hashlib
import random
import string
import uuid

import numpy as np
import pytest
import torch

from cachegen_amd.cache_engine import LMCacheEngine, LMCacheEngineBuilder
from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
from cachegen_amd.storage_backend import (CreateStorageBackend, LMCHybridBackend, LMCLocalBackend,
                                          LMCRemoteBackend)
from cachegen_amd.storage_backend.connector import CreateConnector, InMemoryConnector
from cachegen_amd.utils import CacheEngineKey


def dumb_metadata(fmt="vllm"):
    return LMCacheEngineMetadata("test_model", 3, 123, fmt)


def generate_kv_cache(num_tokens, fmt, device, num_layers=4, num_heads=2, head_size=16, seed=0):
    gen = torch.Generator().manual_seed(seed)
    shape = [num_tokens, num_heads, head_size] if fmt == "vllm" else [num_heads, num_tokens, head_size]
    dtype = torch.bfloat16 if fmt == "vllm" else torch.float16
    return tuple((torch.rand(shape, generator=gen).to(dtype).to(device), torch.rand(shape, generator=gen).to(dtype).to(device))
                 for _ in range(num_layers))


def generate_tokens(num_tokens, device, seed=0):
    gen = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, 10000, size=[num_tokens], generator=gen).to(device)


def concatenate_kv_caches(kv_chunks, fmt):
    dim = 1 if fmt == "huggingface" else 0
    return tuple((torch.cat([c[i][0] for c in kv_chunks], dim=dim), torch.cat([c[i][1] for c in kv_chunks], dim=dim))
                 for i in range(len(kv_chunks[0])))


def check_kv_cache_equal(left, right, num_tokens, fmt):
    dim = 0 if fmt == "vllm" else 1
    assert len(left) == len(right)
    for (lk, lv), (rk, rv) in zip(left, right):
        for a, b in ((lk, rk), (lv, rv)):
            assert a.dim() == 3 and b.dim() == 3
            assert a.shape[dim] >= num_tokens and b.shape[dim] >= num_tokens
            assert torch.equal(a.narrow(dim, 0, num_tokens).cpu(), b.narrow(dim, 0, num_tokens).cpu())


def backend_config(backend, chunk_size=256, serde="torch"):
    if backend == "mem":
        backend = "mem://%s:0" % uuid.uuid4().hex
    return LMCacheEngineConfig.from_legacy(chunk_size=chunk_size, backend=backend, remote_serde=serde)


# --------------------------------------------------------------------------- #
# keys, hashes, configuration
# --------------------------------------------------------------------------- #
def test_key_string_round_trip_and_hashing():
    key = CacheEngineKey("vllm", "org/model", 3, 7, "ab" * 32)
    assert key.to_string() == "vllm@org/model@3@7@" + "ab" * 32
    assert CacheEngineKey.from_string(key.to_string()) == key
    assert hash(key) == hash(CacheEngineKey.from_string(key.to_string()))
    with pytest.raises(ValueError):
        CacheEngineKey.from_string("a@b@c")


def test_prefix_hash_known_answer():
    """Chunk hashes chain: sha256(previous hex digest + the chunk's int64 token ids)."""
    engine = LMCacheEngine(backend_config("cpu", chunk_size=4), dumb_metadata())
    tokens = torch.arange(10, dtype=torch.int64)
    got = list(engine._prefix_hashes(tokens))
    h0 = hashlib.sha256(b"" + np.arange(0, 4, dtype=np.int64).tobytes()).hexdigest()
    h1 = hashlib.sha256(h0.encode("ascii") + np.arange(4, 8, dtype=np.int64).tobytes()).hexdigest()
    h2 = hashlib.sha256(h1.encode("ascii") + np.arange(8, 10, dtype=np.int64).tobytes()).hexdigest()
    assert got == [h0, h1, h2]
    assert engine._make_key(h0, "vllm") == CacheEngineKey("vllm", "test_model", 3, 123, h0)


def test_config_constructors(tmp_path):
    c = LMCacheEngineConfig.from_legacy(chunk_size=128, backend="cuda")
    assert (c.chunk_size, c.local_device, c.remote_url) == (128, "cuda", None)
    c = LMCacheEngineConfig.from_legacy(backend="redis://localhost:6379", remote_serde="cachegen")
    assert (c.local_device, c.remote_url, c.remote_serde) == (None, "redis://localhost:6379", "cachegen")
    f = tmp_path / "cfg.yaml"
    f.write_text("chunk_size: 512\nlocal_device: cpu\nremote_url: mem://x:0\npipelined_backend: true\n")
    c = LMCacheEngineConfig.from_file(str(f))
    assert c == LMCacheEngineConfig(512, "cpu", "mem://x:0", "torch", True)


def test_backend_creation():
    meta = LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, -1, "vllm")
    url = "mem://%s:0" % uuid.uuid4().hex
    local = CreateStorageBackend(LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=None), meta)
    remote = CreateStorageBackend(LMCacheEngineConfig.from_defaults(local_device=None, remote_url=url), meta)
    hybrid = CreateStorageBackend(LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=url), meta)
    assert isinstance(local, LMCLocalBackend) and isinstance(remote, LMCRemoteBackend)
    assert isinstance(hybrid, LMCHybridBackend)
    with pytest.raises(ValueError):
        CreateStorageBackend(LMCacheEngineConfig.from_defaults(local_device=None, remote_url=None), meta)
    with pytest.raises(ValueError):
        CreateConnector("nothing")
    with pytest.raises(ValueError):
        CreateConnector("lm://localhost:65000")
    for b in (local, remote, hybrid):
        b.close()


def test_connector_contract():
    name = uuid.uuid4().hex
    a, b = CreateConnector(f"mem://{name}:0"), CreateConnector(f"mem://{name}:0")
    assert not a.exists("k") and a.get("k") is None and a.list() == []
    a.set("k", b"\x00\x01payload")
    assert b.exists("k") and b.get("k") == b"\x00\x01payload" and b.list() == ["k"]
    InMemoryConnector.drop(name)
    assert not CreateConnector(f"mem://{name}:0").exists("k")


def random_key():
    letters = string.ascii_uppercase + string.digits
    return CacheEngineKey(random.choice(["vllm", "huggingface"]), "".join(random.choices(letters, k=10)), 3,
                          random.randint(0, 100), "".join(random.choices(letters, k=64)))


@pytest.mark.parametrize("kind", ["local", "remote", "hybrid", "hybrid_pipelined"])
@pytest.mark.parametrize("blocking", [True, False])
def test_backends_put_get(kind, blocking):
    url = "mem://%s:0" % uuid.uuid4().hex
    config = {
        "local": LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=None),
        "remote": LMCacheEngineConfig.from_defaults(local_device=None, remote_url=url),
        "hybrid": LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=url),
        "hybrid_pipelined": LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=url, pipelined_backend=True),
    }[kind]
    backend = CreateStorageBackend(config, LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, -1, "vllm"))
    keys = [random_key() for _ in range(6)]
    values = [torch.rand((4, 2, 32, 2, 16)) for _ in keys]
    for key, value in zip(keys, values):
        backend.put(key, value, blocking=blocking)
    remote = getattr(backend, "remote_store", backend)
    if hasattr(remote, "flush"):
        remote.flush()
    assert not backend.contains(random_key())
    for key, value in zip(keys, values):
        assert backend.contains(key)
        assert torch.equal(backend.get(key), value)
    got = list(backend.batched_get(keys[:2] + [random_key()] + keys[2:3]))
    assert torch.equal(got[0], values[0]) and torch.equal(got[1], values[1]) and got[2] is None
    backend.close()


def test_hybrid_backend_prefetches_what_the_remote_side_holds():
    url = "mem://%s:0" % uuid.uuid4().hex
    meta = LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, 5, "vllm")
    config = LMCacheEngineConfig.from_defaults(local_device="cpu", remote_url=url)
    first = CreateStorageBackend(config, meta)
    mine = CacheEngineKey("vllm", meta.model_name, 1, 5, "a" * 64)
    other = CacheEngineKey("vllm", meta.model_name, 1, 6, "b" * 64)          # another worker's chunk
    first.put(mine, torch.ones(3, 3))
    first.put(other, torch.zeros(3, 3))
    second = CreateStorageBackend(config, meta)
    assert second.local_store.contains(mine) and not second.local_store.contains(other)
    assert second.contains(other) and torch.equal(second.get(other), torch.zeros(3, 3))
    first.close()
    second.close()


# --------------------------------------------------------------------------- #
# engine behaviours (test_cache_engine.py of the reference), CPU stores
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("backend", ["cpu", "mem"])
def test_same_retrive_store(fmt, backend):
    num_tokens = 2000
    tokens = generate_tokens(num_tokens, "cpu")
    kv_cache = generate_kv_cache(num_tokens, fmt, "cpu")
    engine = LMCacheEngine(backend_config(backend), dumb_metadata(fmt))
    retrived, length = engine.retrive(tokens, "cpu")
    assert len(retrived) == 0 and length == 0
    engine.store(tokens, kv_cache)
    retrived, length = engine.retrive(tokens, "cpu")
    assert length == num_tokens
    check_kv_cache_equal(retrived, kv_cache, num_tokens, fmt)
    engine.close()


@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("chunk_size", [128, 256])
@pytest.mark.parametrize("backend", ["cpu", "mem"])
def test_retrive_prefix_and_mixed(fmt, chunk_size, backend):
    num_tokens, new_num_tokens = 2000, 1000
    tokens, new_tokens = generate_tokens(num_tokens, "cpu"), generate_tokens(new_num_tokens, "cpu", seed=1)
    kv_cache = generate_kv_cache(num_tokens, fmt, "cpu")
    new_kv_cache = generate_kv_cache(new_num_tokens, fmt, "cpu", seed=1)
    engine = LMCacheEngine(backend_config(backend, chunk_size), dumb_metadata(fmt))
    engine.store(tokens, kv_cache)
    # only whole chunks of the stored prefix come back
    expected_length = num_tokens // chunk_size * chunk_size
    retrived, length = engine.retrive(torch.cat([tokens, new_tokens]), "cpu")
    assert length == expected_length
    check_kv_cache_equal(retrived, kv_cache, expected_length, fmt)
    # a second context does not disturb the first
    engine.store(new_tokens, new_kv_cache)
    retrived, length = engine.retrive(torch.cat([tokens, new_tokens]), "cpu")
    assert length == expected_length
    retrived, length = engine.retrive(new_tokens, "cpu")
    assert length == new_num_tokens
    check_kv_cache_equal(retrived, new_kv_cache, length, fmt)
    # the combined context: its first chunks exist and are kept, the rest is added
    final_tokens = torch.cat([tokens, new_tokens])
    final_kv = concatenate_kv_caches([kv_cache, generate_kv_cache(new_num_tokens, fmt, "cpu", seed=2)], fmt)
    engine.store(final_tokens, final_kv)
    retrived, length = engine.retrive(final_tokens, "cpu")
    assert length == num_tokens + new_num_tokens
    check_kv_cache_equal(retrived, final_kv, length, fmt)
    engine.close()


def test_skip_existing_keeps_and_overwrite_replaces():
    fmt = "vllm"
    tokens = generate_tokens(600, "cpu")
    first, second = generate_kv_cache(600, fmt, "cpu", seed=3), generate_kv_cache(600, fmt, "cpu", seed=4)
    engine = LMCacheEngine(backend_config("cpu"), dumb_metadata(fmt))
    engine.store(tokens, first)
    engine.store(tokens, second, skip_existing=True)
    check_kv_cache_equal(engine.retrive(tokens, "cpu")[0], first, 600, fmt)
    engine.store(tokens, second, skip_existing=False)
    check_kv_cache_equal(engine.retrive(tokens, "cpu")[0], second, 600, fmt)
    # the store holds copies: changing the caller's tensors afterwards changes nothing
    second[0][0].zero_()
    assert engine.retrive(tokens, "cpu")[0][0][0].abs().sum() > 0
    with pytest.raises(AssertionError):
        engine.store(tokens[:-1], second)
    with pytest.raises(AssertionError):
        engine.store(tokens, ())
    engine.close()


def test_nonblocking_store_reaches_the_remote_side():
    fmt = "huggingface"
    tokens, kv_cache = generate_tokens(700, "cpu"), generate_kv_cache(700, fmt, "cpu")
    engine = LMCacheEngine(backend_config("mem"), dumb_metadata(fmt))
    engine.store(tokens, kv_cache, blocking=False)
    engine.engine_.flush()
    retrived, length = engine.retrive(tokens, "cpu")
    assert length == 700
    check_kv_cache_equal(retrived, kv_cache, 700, fmt)
    engine.close()


def test_builder():
    instance_id = "test-" + uuid.uuid4().hex
    cfg, cfg2 = backend_config("cpu", 256), backend_config("cpu", 512)
    assert LMCacheEngineBuilder.get(instance_id) is None
    engine = LMCacheEngineBuilder.get_or_create(instance_id, cfg, dumb_metadata())
    assert LMCacheEngineBuilder.get(instance_id) is engine
    assert LMCacheEngineBuilder.get_or_create(instance_id, cfg, dumb_metadata()) is engine
    with pytest.raises(ValueError):
        LMCacheEngineBuilder.get_or_create(instance_id, cfg2, dumb_metadata())
    with pytest.raises(ValueError):
        LMCacheEngineBuilder.get_or_create(instance_id, cfg, dumb_metadata("huggingface"))
    engine.close()


# --------------------------------------------------------------------------- #
# GPU: local store on the device, and the compressing serdes behind the remote store
# --------------------------------------------------------------------------- #
@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
def test_gpu_local_store(fmt):
    tokens, kv_cache = generate_tokens(1000, "cuda"), generate_kv_cache(1000, fmt, "cuda")
    engine = LMCacheEngine(backend_config("cuda"), dumb_metadata(fmt))
    engine.store(tokens, kv_cache)
    retrived, length = engine.retrive(tokens, "cuda")
    assert length == 1000 and retrived[0][0].is_cuda
    check_kv_cache_equal(retrived, kv_cache, 1000, fmt)
    engine.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("serde", ["cachegen", "cachegen-flat"])
@pytest.mark.parametrize("blocking", [True, False])
def test_gpu_compressing_store_equals_the_serializer_round_trip(fmt, serde, blocking):
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import CreateSerde
    meta = LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, 0, fmt)
    config = backend_config("mem", 256, serde)
    num_tokens = 700
    blob = make_kv(32, num_tokens, 2, 64, seed=17, device="cuda:0")          # [L, 2, T, H, D]
    if fmt == "huggingface":
        blob = blob.permute(0, 1, 3, 2, 4).contiguous()
    kv_cache = tuple((layer[0], layer[1]) for layer in blob)
    tokens = generate_tokens(num_tokens, "cuda")
    engine = LMCacheEngine(config, meta)
    engine.store(tokens, kv_cache, blocking=blocking)
    engine.engine_.flush()
    retrived, length = engine.retrive(tokens, "cuda")
    assert length == num_tokens and len(retrived) == 32
    # the same chunks through the plain per-chunk interface of the reference
    s, d = CreateSerde(serde, config, meta)
    tdim = 2 if fmt == "vllm" else 3
    want = torch.cat([d.from_bytes(s.to_bytes(blob.narrow(tdim, t0, min(256, num_tokens - t0))))
                      for t0 in range(0, num_tokens, 256)], dim=tdim)
    got = torch.stack([torch.stack(pair) for pair in retrived])
    assert got.dtype == want.dtype and torch.equal(got, want)
    # a longer query returns the stored prefix only, a diverging one only its common chunks
    longer = torch.cat([tokens, generate_tokens(300, "cuda", seed=5)])
    assert engine.retrive(longer, "cuda")[1] == 512
    other = tokens.clone()
    other[300] += 1
    assert engine.retrive(other, "cuda")[1] == 256
    # stored blobs are what the serializer gives for each chunk on its own
    remote = engine.engine_
    for i, chunk_hash in enumerate(engine._prefix_hashes(tokens)):
        stored = remote.get_bytes(engine._make_key(chunk_hash, fmt))
        piece = blob.narrow(tdim, 256 * i, min(256, num_tokens - 256 * i))
        alone = s.to_bytes(piece)
        if serde == "cachegen-flat":
            assert stored == alone
        else:
            assert torch.equal(d.from_bytes(stored), d.from_bytes(alone))
    engine.close()
