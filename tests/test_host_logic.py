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


def _sample_container():
    import torch
    from cachegen_amd.serde import cachegen_basics as B
    g = torch.Generator().manual_seed(1)
    chunk = B.CacheGenGPUBytestream(torch.randint(0, 256, (37,), generator=g, dtype=torch.uint8),
                                    torch.randint(0, 9, (4, 3), generator=g, dtype=torch.int32), 7)
    return B.CacheGenGPUEncoderOutput([chunk], torch.randint(-9, 9, (4, 3, 5), generator=g, dtype=torch.int16),
                                      torch.randn((2, 7, 1), generator=g).to(torch.bfloat16),
                                      torch.randn((2, 14, 1), generator=g).to(torch.float16)[:, ::2], 8, 128)


def _same_container(a, b):
    import torch
    assert (a.num_heads, a.head_size, len(a.data_chunks)) == (b.num_heads, b.head_size, len(b.data_chunks))
    for x, y in zip(a.data_chunks, b.data_chunks):
        assert x.ntokens == y.ntokens and torch.equal(x.bytestream, y.bytestream)
        assert torch.equal(x.bytestream_lengths, y.bytestream_lengths)
    for f in ("cdf", "max_tensors_key", "max_tensors_value"):
        assert a[f].dtype == b[f].dtype and torch.equal(a[f], b[f])


def test_container_reads_a_blob_pickled_under_the_references_module_path():
    """The reference pickles `lmcache.storage_backend.serde.cachegen_basics.CacheGenGPUEncoderOutput`
    (cachegen_basics.py:133-156).  Such a blob is made here by pickling this package's own classes
    while they claim that module path; no reference code is imported."""
    from cachegen_amd.serde import cachegen_basics as B
    obj = _sample_container()
    mine = obj.to_bytes()
    _same_container(B.CacheGenGPUEncoderOutput.from_bytes(mine), obj)

    # pickle with the classes temporarily claiming the reference's module path
    saved = {c: c.__module__ for c in (B.CacheGenGPUEncoderOutput, B.CacheGenGPUBytestream)}
    import sys
    import types
    ref_name = "lmcache.storage_backend.serde.cachegen_basics"
    # pickle checks that module.name is the object it writes: empty stand-in modules, for the
    # length of the dump only
    parts = ref_name.split(".")
    names = [".".join(parts[:i + 1]) for i in range(len(parts))]
    assert not any(n in sys.modules for n in names)
    try:
        for n in names:
            sys.modules[n] = types.ModuleType(n)
        sys.modules[ref_name].CacheGenGPUEncoderOutput = B.CacheGenGPUEncoderOutput
        sys.modules[ref_name].CacheGenGPUBytestream = B.CacheGenGPUBytestream
        for c in saved:
            c.__module__ = ref_name
        theirs = obj.to_bytes()
    finally:
        for c, m in saved.items():
            c.__module__ = m
        for n in names:
            sys.modules.pop(n, None)
    assert ref_name.encode() in theirs and b"cachegen_amd" not in theirs
    assert ref_name not in sys.modules
    _same_container(B.CacheGenGPUEncoderOutput.from_bytes(theirs), obj)


def test_container_refuses_any_other_global():
    import pickle
    import pytest
    from cachegen_amd.serde import cachegen_basics as B
    for evil in (pickle.dumps(print), pickle.dumps(__import__("os").system),
                 b"cbuiltins\neval\n(V1+1\ntR."):
        with pytest.raises(pickle.UnpicklingError, match="refusing to load"):
            B.CacheGenGPUEncoderOutput.from_bytes(evil)


def test_built_kernels_keep_their_register_budget():
    """The stream kernels need eight wavefronts per SIMD and no scratch memory; the build writes
    the compiler's figures beside the library and refuses a library that breaks a budget.  This
    reads the figures of the library the other tests load."""
    import json
    import os
    from cachegen_amd import build
    assert os.path.exists(build.RESOURCES), "build the library with cachegen_amd.build.build_library()"
    assert os.path.getmtime(build.RESOURCES) >= os.path.getmtime(build.LIBRARY) - 120, "resource report older than the library"
    with open(build.RESOURCES) as f:
        resources = json.load(f)
    build.check_budgets(resources)
    fused = resources["encode_streams_kernel<256, true, true, false, true, true>"]
    assert fused["vgprs"] <= 64 and fused["scratch"] == 0 and fused["occupancy"] == 8
    # the check does fail when a kernel crosses the line
    import pytest
    broken = dict(resources)
    broken["encode_streams_kernel<256, true, true, false, true, true>"] = dict(fused, vgprs=72, occupancy=7)
    with pytest.raises(RuntimeError, match="budget 8"):
        build.check_budgets(broken)
    spilled = dict(resources)
    spilled["compact_streams_kernel<true>"] = dict(resources["compact_streams_kernel<true>"], scratch=16)
    with pytest.raises(RuntimeError, match="scratch"):
        build.check_budgets(spilled)


def test_probe_library_loads_and_exports_its_entry_points():
    from cachegen_amd import issue_probe
    h = issue_probe.lib()
    for name in ("cg_probe_issue_rate", "cg_probe_clock_start", "cg_probe_clock_result"):
        assert hasattr(h, name)
