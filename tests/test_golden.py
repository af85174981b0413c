"""Golden fixtures (tests/golden): hand-derived known answers and a seeded regression vector.
CPU tests check the oracle against them; GPU tests check the HIP path against the same files
without going through the oracle."""
import json
import os

import numpy as np
import pytest
import torch

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KA = json.load(open(os.path.join(HERE, "known_answers.json")))
DEV = "cuda:0"


def _reg():
    return np.load(os.path.join(HERE, "regression_kv.npz"))


# ---------------------------------------------------------------- oracle vs fixtures (CPU)
def test_oracle_known_answers(oracle):
    for k in KA["quantize"]:
        x = np.array([[k["row"]]], dtype=np.float16)
        sym, mx = oracle.quantize(x.view(np.uint16), [float(k["bins"])])
        assert sym[0, 0].tolist() == k["symbols"] and float(mx.view(np.float16)[0, 0]) == k["max"]
    for k in KA["cdf"]:
        sym = np.array(k["symbols"], dtype=np.uint8).reshape(1, -1, 1)
        assert oracle.calculate_cdf(sym, k["max_bins"])[0, 0].tolist() == k["cdf"]
    for k in KA["coder"]:
        data, n = oracle.encode_stream(k["cdf"], k["symbols"])
        assert list(data) == k["bytes"] and n == len(k["bytes"])
        assert oracle.decode_stream(k["cdf"], bytes(k["bytes"]), len(k["symbols"])).tolist() == k["symbols"]
    for k in KA["decoder_boundary"]:
        assert oracle.decode_stream(k["cdf"], bytes(k["bytes"]), len(k["symbols"])).tolist() == k["symbols"]
    for k in KA["dequantize"]:
        out = oracle.dequantize(np.array([[k["symbols"]]], dtype=np.uint8), [float(k["bins"])],
                                np.array([[k["max"]]], dtype=np.float16).view(np.uint16))
        assert out[0, 0].tolist() == k["float16_bits"]


def test_oracle_reproduces_regression_fixture(oracle):
    r = _reg()
    enc = oracle.encode_function(r["kv_bits"], r["key_bins"], r["value_bins"])
    assert np.array_equal(enc["cdf"], r["cdf"])
    assert np.array_equal(enc["max_tensors_key"], r["max_key"])
    assert np.array_equal(np.stack([c[1] for c in enc["data_chunks"]]), r["lengths"])
    assert np.array_equal(np.concatenate([c[0] for c in enc["data_chunks"]]), r["payload"])
    _, out = oracle.decode_function(enc, r["key_bins"], r["value_bins"])
    assert np.array_equal(out, r["dequantized_f16_bits"])


# ---------------------------------------------------------------- HIP path vs fixtures (GPU)
@pytest.mark.gpu
def test_hip_known_answers():
    from cachegen_amd import codec, torchac_hip as tac
    for k in KA["quantize"]:
        row = k["row"] * 2                                  # 8 channels: the vector path
        x = torch.tensor(row, dtype=torch.float16).view(1, 1, 1, 1, 8)
        kv = torch.cat([x, x], dim=1).to(DEV)
        b = torch.tensor([float(k["bins"])], device=DEV)
        sym, mx = codec.quantize_kv(kv, b, b)
        assert sym[0, 0].tolist() == k["symbols"] * 2 and float(mx[0, 0, 0]) == k["max"]
    for k in KA["cdf"]:
        sym = torch.tensor(k["symbols"], dtype=torch.int8, device=DEV).view(1, -1, 1)
        got = tac.calculate_cdf(sym, k["max_bins"]).cpu().numpy().view(np.uint16)[0, 0].tolist()
        assert got == k["cdf"]
    for k in KA["coder"]:
        cdf = torch.tensor(np.array(k["cdf"], dtype=np.uint16).view(np.int16), device=DEV).view(1, 1, -1)
        sym = torch.tensor(k["symbols"], dtype=torch.int8, device=DEV).view(1, -1, 1)
        out = torch.zeros((1, 1, 256), dtype=torch.uint8, device=DEV)
        lens = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
        tac.encode_fast_new(cdf, sym, out, lens)
        assert int(lens) == len(k["bytes"]) and out[0, 0, :len(k["bytes"])].tolist() == k["bytes"]
        if k["symbols"]:
            back = torch.zeros((1, len(k["symbols"]), 1), dtype=torch.uint8, device=DEV)
            tac.decode_fast_new(cdf, out, lens, back)
            assert back.flatten().tolist() == k["symbols"]
    for k in KA["decoder_boundary"]:
        cdf = torch.tensor(np.array(k["cdf"], dtype=np.uint16).view(np.int16), device=DEV).view(1, 1, -1)
        n = len(k["symbols"])
        data = torch.tensor(k["bytes"], dtype=torch.uint8, device=DEV)
        back = torch.zeros((1, n, 1), dtype=torch.uint8, device=DEV)
        prefix = torch.tensor([[len(k["bytes"])]], dtype=torch.int64, device=DEV)
        tac.decode_fast_prefsum(cdf, data, prefix, back)
        assert back.flatten().tolist() == k["symbols"]
        padded = torch.zeros((1, 1, 256), dtype=torch.uint8, device=DEV)
        padded[0, 0, :len(k["bytes"])] = data
        back2 = torch.zeros((1, n, 1), dtype=torch.uint8, device=DEV)
        tac.decode_fast_new(cdf, padded, torch.tensor([[len(k["bytes"])]], dtype=torch.int32, device=DEV), back2)
        assert back2.flatten().tolist() == k["symbols"]


@pytest.mark.gpu
def test_hip_reproduces_regression_fixture():
    from cachegen_amd import codec
    r = _reg()
    L, _, T, C = r["kv_bits"].shape
    kv = torch.from_numpy(r["kv_bits"].view(np.int16)).view(torch.float16).view(L, 2, T, 2, C // 2).to(DEV)
    kb = torch.from_numpy(r["key_bins"]).to(DEV)
    vb = torch.from_numpy(r["value_bins"]).to(DEV)
    enc = codec.encode_kv(kv, kb, vb, chunk_tokens=T)
    enc.check()
    assert np.array_equal(enc.cdf[0].cpu().numpy().view(np.uint16), r["cdf"])
    assert np.array_equal(enc.lengths.cpu().numpy(), r["lengths"])
    n = enc.total_bytes()
    assert np.array_equal(enc.payload[:n].cpu().numpy(), r["payload"])
    assert np.array_equal(enc.maxima[0].cpu().view(torch.int16).numpy().view(np.uint16), r["max_key"])
    out = codec.decode_encoded(enc, kb, vb, fmt="vllm", out_dtype=torch.float16)
    got = out.cpu().view(torch.int16).numpy().view(np.uint16).reshape(L, 2, T, C)
    assert np.array_equal(got, r["dequantized_f16_bits"])
