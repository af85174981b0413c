"""Adaptive streaming (cachegen_amd/adaptive.py): the controller's decisions on the CPU
(src/utils.py:294-317 restated on blob sizes), and on the GPU the multi-level encode and the
in-place reassembly against the per-chunk deserializer."""
import json
import os
import random

import numpy as np
import pytest
import torch

from cachegen_amd import adaptive

HERE = os.path.dirname(os.path.abspath(__file__))


def test_config_selection_known_answer():
    # slo 2 s over 3 chunks: 0.6667 s each
    sizes = [{1: 40_000_000, 2: 60_000_000, 3: 90_000_000}] * 3
    ttft, configs = adaptive.config_selection([1.0, 0.05, 8.0], chunk_delay=0.2, slo=2.0, chunk_size=1000,
                                              length=3000, blob_sizes=sizes)
    # chunk 0 at 1 Gbps: level 3 takes 0.72 s (too long), level 2 takes 0.48 s
    # chunk 1 at 0.05 Gbps: even level 1 takes 6.4 s -> recomputed for 0.2 s
    # chunk 2 at 8 Gbps: level 3 takes 0.09 s
    assert configs == [2, 0, 3]
    assert ttft == pytest.approx(0.48 + 0.2 + 0.09, rel=1e-12)


def test_config_selection_budget_is_strict_and_tail_chunk_counts():
    # exactly on the budget is not good enough (strict "<" at src/utils.py:306)
    sizes = [{1: 1, 2: 125_000_000, 3: 125_000_000}]
    ttft, configs = adaptive.config_selection([1.0], 0.2, slo=1.0, chunk_size=1000, length=1000, blob_sizes=sizes)
    assert configs == [1]
    # 2500 tokens: round(2.5) = 2 shares of the SLO, but three chunks are visited
    sizes = [{1: 10, 2: 20, 3: 30}] * 3
    ttft, configs = adaptive.config_selection([1.0, 1.0, 1.0], 0.2, slo=2.0, chunk_size=1000, length=2500,
                                              blob_sizes=sizes)
    assert configs == [3, 3, 3] and ttft == pytest.approx(3 * 30 * 8e-9)
    with pytest.raises(IndexError):
        adaptive.config_selection([1.0, 1.0], 0.2, 2.0, 1000, 2500, sizes)


def test_config_selection_on_the_reference_bandwidth_traces():
    """Three of the traces the reference ships (test_data/bw.jsonl): the result obeys the
    controller's defining properties on each."""
    traces = json.load(open(os.path.join(HERE, "golden", "bw_traces.json")))
    sizes = [{1: 60_000_000, 2: 110_000_000, 3: 160_000_000}] * 10
    for trace in traces:
        bws = trace["bw"]
        assert len(bws) == 10
        ttft, configs = adaptive.config_selection(bws, 0.2, slo=2.0, chunk_size=1000, length=10_000,
                                                  blob_sizes=sizes)
        assert len(configs) == 10
        total = 0.0
        for bw, level in zip(bws, configs):
            times = {lv: sizes[0][lv] * 8e-9 / bw for lv in (1, 2, 3)}
            fitting = [lv for lv in (3, 2, 1) if times[lv] < 0.2]
            assert level == (fitting[0] if fitting else 0)
            total += times[level] if level else 0.2
        assert ttft == pytest.approx(total, rel=1e-12)
    # first trace, by hand: 0.566 Gbps fits nothing (level 1 needs 0.848 s); 5.03 Gbps fits level 2
    # (0.175 s) but not level 3 (0.255 s)
    _, configs = adaptive.config_selection(traces[0]["bw"], 0.2, 2.0, 1000, 10_000, sizes)
    assert configs[:2] == [0, 2]


def test_bw_generator_range_and_seed():
    a = adaptive.bw_generator(50, random.Random(7))
    b = adaptive.bw_generator(50, random.Random(7))
    assert a.shape == (50,) and np.array_equal(a, b) and a.min() >= 0.1 and a.max() <= 10


def test_level_bins_follow_the_reference_table_and_leave_the_environment_alone(monkeypatch):
    monkeypatch.setenv("QUANT_LEVEL", "3")
    k1, v1 = adaptive.level_bins(1)
    assert os.environ["QUANT_LEVEL"] == "3"
    assert k1.tolist() == [16.0] * 20 + [12.0] * 12 and v1.tolist() == [16.0] * 2 + [12.0] * 30
    k3, v3 = adaptive.level_bins(3)
    assert k3.tolist() == [32.0] * 32 and v3.tolist() == [32.0] * 32
    monkeypatch.delenv("QUANT_LEVEL")
    k2, _ = adaptive.level_bins(2)
    assert "QUANT_LEVEL" not in os.environ and k2.tolist() == [32.0] * 10 + [16.0] * 22
    with pytest.raises(ValueError):
        adaptive.level_bins(7)


def test_tuple_and_blob_round_trip():
    kv = torch.arange(2 * 2 * 3 * 4 * 5, dtype=torch.float32).reshape(2, 2, 3, 4, 5)
    tup = adaptive.tensor_to_tuple(kv)
    assert len(tup) == 2 and tup[1][0].shape == (1, 3, 4, 5)
    back = adaptive.to_blob([(k[0], v[0]) for k, v in tup], device="cpu")
    assert torch.equal(back, kv)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
def test_levels_encode_and_merge_match_the_per_chunk_deserializer(fmt, monkeypatch):
    from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import CreateSerde
    chunk, T = 256, 700
    kv = make_kv(32, T, 2, 64, seed=21, device="cuda:0")
    if fmt == "huggingface":
        kv = kv.permute(0, 1, 3, 2, 4).contiguous()
    tdim = 2 if fmt == "vllm" else 3
    blobs = adaptive.encode_levels(kv, chunk, fmt=fmt)
    assert len(blobs) == 3 and all(sorted(b) == [1, 2, 3] for b in blobs)
    for b in blobs:
        assert len(b[1]) < len(b[2]) < len(b[3])

    sizes = [{lv: len(b[lv]) for lv in b} for b in blobs]
    # bandwidths chosen so that the three chunks get levels 3, 0 and 1
    budget = 1.0 / round(T / chunk)
    bws = [sizes[0][3] * 8e-9 / budget * 1.01, sizes[1][1] * 8e-9 / budget * 0.5,
           sizes[2][1] * 8e-9 / budget * 1.01]
    ttft, configs = adaptive.config_selection(bws, 0.05, 1.0, chunk, T, sizes)
    assert configs == [3, 0, 1]

    out_dtype = torch.bfloat16 if fmt == "vllm" else torch.float16      # what the deserializer returns
    merged = adaptive.merge(configs, blobs, chunk, T, orig_kv=kv, fmt=fmt, out_dtype=out_dtype)
    want_shape = list(kv.shape)
    want_shape[tdim] = 512                                     # the 188-token tail is dropped
    assert list(merged.shape) == want_shape and merged.dtype == out_dtype
    assert adaptive.merge(configs, blobs, chunk, T, orig_kv=kv, fmt=fmt).dtype == kv.dtype
    meta = LMCacheEngineMetadata("mistralai/Mistral-7B-Instruct-v0.2", 1, 0, fmt)
    config = LMCacheEngineConfig.from_defaults(chunk_size=chunk)
    for chunk_id, level in enumerate(configs[:2]):
        got = merged.narrow(tdim, chunk_id * chunk, chunk)
        piece = kv.narrow(tdim, chunk_id * chunk, chunk)
        if level == 0:
            assert torch.equal(got, piece.to(out_dtype))
            continue
        monkeypatch.setenv("QUANT_LEVEL", str(level))
        s, d = CreateSerde("cachegen", config, meta)
        want = d.from_bytes(s.to_bytes(piece))
        assert want.dtype == out_dtype and torch.equal(got, want)
