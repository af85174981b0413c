"""CPU-side checks: the C ABI library loads and exports what the header declares, and the
host logic (bins tables, chunk arithmetic, generator) behaves like the reference's."""
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from cachegen_amd import _lib
    header = open(os.path.join(ROOT, "include", "cachegen_hip.h")).read()
    declared = set(re.findall(r"\b(cg_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 12
    lib = _lib.lib()
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert lib.cg_abi_version() == 5
    assert lib.cg_last_error() == b""


def test_chunk_arithmetic():
    from cachegen_amd import _lib
    lib = _lib.lib()
    assert lib.cg_num_chunks(8192, 256) == 32 and lib.cg_num_subchunks(8192, 256) == 32
    assert lib.cg_num_subchunks(512, 512) == 2
    assert lib.cg_num_chunks(32768, 1500) == 22 and lib.cg_num_subchunks(32768, 1500) == 21 * 6 + 5
    assert lib.cg_num_subchunks(236, 256) == 1 and lib.cg_num_subchunks(257, 1000) == 2
    assert lib.cg_num_subchunks(0, 256) == 0
    assert lib.cg_encode_kv_workspace(2, 512, 512, 512) >= 2 * 2 * 512 * 512 + 2 * 4 * 512 * 256


def test_decode_kv_refuses_output_strides_it_cannot_address():
    """Argument checks only: they come before anything touches a device, so the pointers here
    are never dereferenced."""
    from cachegen_amd import _lib
    lib = _lib.lib()
    fake = 4096
    L, T, H, D = 2, 256, 8, 128

    def call(ot, oh):
        return lib.cg_decode_kv(fake, 32, fake, 0, fake, fake, 1024, fake, fake, L, T, H, D, 256, 0,
                                fake, 0, 2 * T * H * D, T * H * D, ot, oh, None)

    assert call(-H * D, D) != 0 and b"strides" in lib.cg_last_error()
    assert call(H * D, -D) != 0
    assert call(1 << 24, D) != 0 and b"4 GiB" in lib.cg_last_error()         # 255 rows of 32 MiB
    assert call(D, 1 << 29) != 0                                           # heads 1 GiB apart


def test_bins_tables_match_reference_tables(monkeypatch):
    from cachegen_amd.serde.cachegen_basics import CacheGenConfig, make_key_bins, make_value_bins
    cfg = CacheGenConfig.from_model_name("lmsys/longchat-7b-16k")
    assert make_key_bins(cfg).tolist() == [32.0] * 10 + [16.0] * 22
    assert make_value_bins(cfg).tolist() == [32.0] * 2 + [16.0] * 30
    cfg = CacheGenConfig.from_model_name("Yukang/LongAlpaca-70B-16k")
    assert make_key_bins(cfg).tolist() == [32.0] * 40 + [16.0] * 40
    assert make_value_bins(cfg).tolist() == [32.0] * 20 + [16.0] * 60
    monkeypatch.delenv("QUANT_LEVEL", raising=False)
    with pytest.raises(KeyError):
        CacheGenConfig.from_model_name("mistralai/Mistral-7B-Instruct-v0.2")
    monkeypatch.setenv("QUANT_LEVEL", "1")
    cfg = CacheGenConfig.from_model_name("mistralai/Mistral-7B-Instruct-v0.2")
    assert make_key_bins(cfg).tolist() == [16.0] * 20 + [12.0] * 12
    assert make_value_bins(cfg).tolist() == [16.0] * 2 + [12.0] * 30
    monkeypatch.setenv("QUANT_LEVEL", "3")
    assert make_key_bins(CacheGenConfig.from_model_name("x/Mistral-7B-y")).tolist() == [32.0] * 32
    monkeypatch.setenv("QUANT_LEVEL", "9")
    assert CacheGenConfig.from_model_name("x/Mistral-7B-y") is None
    with pytest.raises(ValueError):
        CacheGenConfig.from_model_name("gpt2")
    assert cfg["key_first_layers"] == 10


def test_serde_factory_rejects_unknown_type():
    from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
    from cachegen_amd.serde import CreateSerde
    with pytest.raises(ValueError):
        CreateSerde("nope", LMCacheEngineConfig.from_defaults(), LMCacheEngineMetadata("m", 1, 0, "vllm"))


def test_generator_is_seeded_and_shaped():
    from cachegen_amd.kvgen import make_kv
    a = make_kv(2, 40, 2, 16, seed=4)
    b = make_kv(2, 40, 2, 16, seed=4)
    c = make_kv(2, 40, 2, 16, seed=5, rho=[0.5, 0.95])
    assert a.shape == (2, 2, 40, 2, 16) and a.dtype == torch.float16
    assert torch.equal(a, b) and not torch.equal(a, c)
    x = make_kv(1, 4000, 1, 8, seed=1, outlier_frac=0.0).float()[0, 0, :, 0, :]
    r = ((x[1:] * x[:-1]).mean(0) / (x * x).mean(0)).mean()
    assert 0.85 < float(r) < 0.95                     # AR(1) with rho = 0.9


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    """No fallback: without the built library every entry of the product path raises."""
    import torch
    from cachegen_amd import _lib, codec
    monkeypatch.setattr(_lib, "_handle", None)
    monkeypatch.setattr(_lib, "LIBRARY", str(tmp_path / "libcachegen_hip.so"))
    with pytest.raises(RuntimeError, match="is missing"):
        _lib.lib()
    with pytest.raises(RuntimeError, match="is missing"):
        codec.num_subchunks(512, 256)
    with pytest.raises(RuntimeError, match="should be on GPU"):
        codec.encode_kv(torch.zeros((1, 2, 4, 1, 8), dtype=torch.float16), torch.ones(1), torch.ones(1))


def test_product_code_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under cachegen_amd/ names it."""
    import os
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cachegen_amd")
    for folder, _, files in os.walk(root):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(folder, name)).read()
                assert "oracle" not in text.replace("no reference to be at parity", ""), os.path.join(folder, name)


def test_decode_kv_refuses_inputs_that_do_not_have_the_geometry():
    """A blob made for a model with more layers than the bins vectors, or tensors of the wrong
    shape, is refused on the host before any kernel could index past a buffer."""
    import torch
    from cachegen_amd import codec
    L, T, H, D, S = 2, 300, 2, 8, 256
    C, nsub = H * D, 2
    cdf = torch.zeros((2, 2 * L, C, 33), dtype=torch.int16)
    maxima = torch.zeros((2, L, T), dtype=torch.float16)
    offsets = torch.zeros(nsub * 2 * L * C + 1, dtype=torch.int64)
    payload = torch.zeros(64, dtype=torch.uint8)
    bins = torch.full((L,), 32.0)

    def call(**kw):
        a = dict(cdf=cdf, maxima=maxima, offsets=offsets, payload=payload, key_bins=bins, value_bins=bins)
        a.update(kw)
        return codec.decode_kv(a["cdf"], a["maxima"], a["offsets"], a["payload"], a["key_bins"], a["value_bins"],
                               L, T, H, D, S, out=torch.empty((L, 2, T, H, D), dtype=torch.float16))
    with pytest.raises(RuntimeError, match="one entry per layer"):
        call(key_bins=torch.full((L - 1,), 32.0))
    with pytest.raises(RuntimeError, match="tables must be"):
        call(cdf=cdf[:1])
    with pytest.raises(RuntimeError, match="tables must be"):
        call(cdf=torch.zeros((2, 2 * L + 2, C, 33), dtype=torch.int16))
    with pytest.raises(RuntimeError, match="row maxima must have shape"):
        call(maxima=maxima[:, :, :-1])
    with pytest.raises(RuntimeError, match="offsets must be"):
        call(offsets=offsets[:-1])
    with pytest.raises(RuntimeError, match="payload must be"):
        call(payload=payload[:0])
