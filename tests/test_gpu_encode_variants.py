"""The internal forms of cg_encode_kv give the same bytes.

Where the tables are built is a choice the library makes by the size of the call: the quantizer
counts the symbols as it makes them (quantize_tables_kernel: torch_quant_vectorized,
encoder.py:42-59, and calculate_cdf, cal_cdf.cu:17-59, in one pass) when the call has (row,
chunk) pairs enough to fill the GPU, else the coder or a separate pass over the symbols does.
The small inputs the oracle can follow would never take the first form by themselves, so the
library's test entry point forces each form here; every form is compared with the oracle.
A call with few (row, chunk) pairs but long chunks (the reference serializer's one table over a
whole context) cuts each chunk into parts counted by separate blocks, whose counters are summed in
memory before the tables are made: SPLIT_CHUNKS forces parts of 256 tokens.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

BYTE_SYMBOLS, TABLES_IN_QUANTIZER, TABLES_IN_CODER, SPLIT_CHUNKS = 1, 2, 4, 8


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _same(a, b):
    n = a.total_bytes()
    assert b.total_bytes() == n
    assert torch.equal(a.cdf, b.cdf), "tables"
    assert torch.equal(a.maxima.view(torch.int16), b.maxima.view(torch.int16)), "maxima"       # as bits: a NaN maximum equals itself
    assert torch.equal(a.lengths, b.lengths), "lengths"
    assert torch.equal(a.offsets, b.offsets), "offsets"
    assert torch.equal(a.payload[:n], b.payload[:n]), "payload"
    assert int(a.status) == int(b.status)


def _against_oracle(oracle, enc, kv, kb, vb, S, dt, fmt="vllm"):
    L, T, H, D = enc.num_layers, enc.num_tokens, enc.num_heads, enc.head_size
    x = kv if fmt == "vllm" else kv.permute(0, 1, 3, 2, 4)
    flat = bits(x).reshape(L, 2, T, H * D)
    bounds = enc.sub_boundaries()
    for ci, c0 in enumerate(range(0, T, S)):
        c1 = min(c0 + S, T)
        want = oracle.encode_function(np.ascontiguousarray(flat[:, :, c0:c1]), kb.numpy(), vb.numpy(), dt)
        cdf, mk, mv, subs = enc.chunk(ci, bounds)
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"]), ("tables", ci)
        assert np.array_equal(bits(mk)[..., 0], want["max_tensors_key"])
        assert np.array_equal(bits(mv)[..., 0], want["max_tensors_value"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert n == wn and np.array_equal(l.cpu().numpy(), wl) and np.array_equal(b.cpu().numpy(), wb)


@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("L,T,H,D,S,bins", [
    (2, 512, 8, 128, 256, (32.0, 16.0)),        # 1024 channels, a table per sub-chunk
    (2, 600, 8, 128, 300, (16.0, 32.0)),        # ragged chunks: 256 + 44 tokens share a table
    (1, 1600, 8, 128, 1500, (32.0,)),           # long chunks: 5 x 256 + 220 tokens under one table
    (3, 300, 4, 64, 300, (32.0, 16.0, 12.0)),   # 256 channels: half the units of a wavefront idle
    (2, 257, 8, 64, 256, (64.0, 32.0)),         # tables of 65 entries; a chunk of one token
    (2, 300, 16, 128, 256, (32.0, 16.0)),       # 2048 channels
    (2, 70, 3, 40, 64, (32.0, 8.0)),            # 120 channels: not a multiple of 64
])
def test_every_form_of_the_encoder_matches_the_oracle(oracle, dtype, dt, L, T, H, D, S, bins):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(L, T, H, D, seed=5 + T + H, dtype=dtype)
    kv[0, 0, 3] = 0                                             # a row of zeros
    kb = torch.tensor(bins)
    vb = torch.tensor(bins[::-1])
    dev = kv.to(DEV)
    plain = codec.encode_kv(dev, kb, vb, chunk_tokens=S)
    plain.check()
    _against_oracle(oracle, plain, kv, kb, vb, S, dt)
    for flags in (TABLES_IN_QUANTIZER, TABLES_IN_CODER, TABLES_IN_QUANTIZER | BYTE_SYMBOLS, TABLES_IN_CODER | BYTE_SYMBOLS,
                  TABLES_IN_QUANTIZER | SPLIT_CHUNKS, TABLES_IN_QUANTIZER | SPLIT_CHUNKS | BYTE_SYMBOLS):
        other = codec.encode_kv(dev, kb, vb, chunk_tokens=S, _test_flags=flags)
        other.check()
        _same(plain, other)
        if flags in (TABLES_IN_QUANTIZER, TABLES_IN_QUANTIZER | SPLIT_CHUNKS):
            _against_oracle(oracle, other, kv, kb, vb, S, dt)


def test_forms_agree_on_the_other_layout_and_on_saturated_rows(oracle):
    """[L,2,H,T,D] storage (heads not contiguous in a token row), bfloat16 rows whose scale
    overflows, a NaN, an infinity and a table shorter than a row's alphabet."""
    from cachegen_amd import codec
    torch.manual_seed(4)
    L, T, H, D = 2, 520, 8, 128
    kv = torch.randn((L, 2, T, H, D), dtype=torch.float32)
    kv[0, 1, 300] *= 1e-39
    kv[1, 0, 0:3] *= 2e-39
    kv[1, 1, 519] *= 1e-39
    kv[0, 0, 17, 2, 5] = float("nan")
    kv[1, 1, 100, 7, 127] = float("inf")
    kv = kv.to(torch.bfloat16)
    kb = torch.tensor([32.0, 16.0])
    vb = torch.tensor([16.0, 32.0])
    hf = kv.permute(0, 1, 3, 2, 4).contiguous().to(DEV)
    for fmt, dev in (("vllm", kv.to(DEV)), ("huggingface", hf)):
        for max_bins in (None, 12):
            base = codec.encode_kv(dev, kb, vb, chunk_tokens=260, fmt=fmt, max_bins=max_bins, _test_flags=TABLES_IN_CODER)
            for flags in (TABLES_IN_QUANTIZER, TABLES_IN_QUANTIZER | BYTE_SYMBOLS, TABLES_IN_QUANTIZER | SPLIT_CHUNKS):
                _same(base, codec.encode_kv(dev, kb, vb, chunk_tokens=260, fmt=fmt, max_bins=max_bins, _test_flags=flags))


def test_default_call_takes_the_quantizer_form_at_benchmark_size():
    """config 2 has 2048 (row, chunk) pairs: cg_encode_kv itself builds the tables in the quantizer
    there; the other form, forced, gives the same bytes for the whole cache."""
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import cachegen_basics as B
    cfg = B.CacheGenConfig.from_model_name("lmsys/longchat-7b-16k")
    kb, vb = B.make_key_bins(cfg).to(DEV), B.make_value_bins(cfg).to(DEV)
    kv = make_kv(32, 8192, 8, 128, seed=1236, device=DEV)
    a = codec.encode_kv(kv, kb, vb, chunk_tokens=256)
    b = codec.encode_kv(kv, kb, vb, chunk_tokens=256, _test_flags=TABLES_IN_CODER)
    a.check()
    _same(a, b)
    # chunks of 1500 tokens: six sub-chunks under one table
    a = codec.encode_kv(kv, kb, vb, chunk_tokens=1500)
    b = codec.encode_kv(kv, kb, vb, chunk_tokens=1500, _test_flags=TABLES_IN_CODER)
    a.check()
    _same(a, b)
    # one table over the whole context, the reference serializer's own call: 64 (row, chunk) pairs,
    # so every chunk is counted in parts of 256 tokens
    a = codec.encode_kv(kv, kb, vb, chunk_tokens=8192)
    b = codec.encode_kv(kv, kb, vb, chunk_tokens=8192, _test_flags=TABLES_IN_CODER)
    a.check()
    _same(a, b)
    # three chunks of 3000 tokens (the last one 2192, so some parts hold no token); and chunks of
    # 1024 tokens: 512 pairs, cut as well
    for S in (3000, 1024):
        a = codec.encode_kv(kv, kb, vb, chunk_tokens=S)
        b = codec.encode_kv(kv, kb, vb, chunk_tokens=S, _test_flags=TABLES_IN_CODER)
        a.check()
        _same(a, b)


def test_largest_call_whose_tile_counts_are_summed_by_groups():
    """16 384 scratch tiles (4 194 304 streams) is the most for which the compaction adds up group
    sums and tile counts itself (256 groups of 64 tiles); one sub-chunk more and a scan launch
    makes the running sum.  Both sides of the line against the form with the tables built in the
    coder, which always runs the scan: same offsets, lengths and payload."""
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import cachegen_basics as B
    cfg = B.CacheGenConfig.from_model_name("lmsys/longchat-7b-16k")
    kb, vb = B.make_key_bins(cfg).to(DEV), B.make_value_bins(cfg).to(DEV)
    kv = make_kv(32, 16384 + 256, 8, 128, seed=77, device=DEV)
    for T in (16384, 16384 + 256):
        x = kv[:, :, :T]
        a = codec.encode_kv(x, kb, vb, chunk_tokens=256)
        b = codec.encode_kv(x, kb, vb, chunk_tokens=256, _test_flags=TABLES_IN_CODER)
        a.check()
        _same(a, b)
        assert int(a.offsets[-1]) == a.total_bytes() == int(a.lengths.sum())
        del a, b

