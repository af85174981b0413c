"""Token rows whose quantization scale overflows, and tables shorter than a row's alphabet.

A bfloat16 row maximum below about 2^-125 makes `MAX / max` infinite (encoder.py:50-55): every
non-zero value of the row saturates.  The reference then reads its shared-memory table at row 255
(enc_new.cu:266-270), far outside the table: undefined there.  This library defines the case: the
saturated byte is the table's last symbol, in the tables and in the streams, and the decoder takes
the same rule.  The checks below feed the oracle's table builder and coder (cal_cdf.cu:17-59,
enc_new.cu:255-317 restated in C) with the symbols clamped that way and require the fused GPU
path to give the same tables, lengths and bytes, for block shapes in which the saturated row lies
beyond the first `block size` token rows of its sub-chunk, and for tables that are shorter than
the alphabet of a row.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _check_against_oracle_on_clamped_symbols(oracle, codec, kv, kb, vb, chunk, max_bins, dt):
    L, _, T, H, D = kv.shape
    C = H * D
    dev = kv.to(DEV)
    enc = codec.encode_kv(dev, kb.to(DEV), vb.to(DEV), chunk_tokens=chunk, max_bins=max_bins)
    enc.check()
    sym, maxima = codec.quantize_kv(dev, kb.to(DEV), vb.to(DEV))
    sym = np.minimum(sym.cpu().numpy(), max_bins - 1)           # the rule: out-of-table bytes are the last symbol
    assert torch.equal(maxima, enc.maxima)
    offs = enc.offsets.cpu().numpy()
    lengths = enc.lengths.cpu().numpy()
    payload = enc.payload.cpu().numpy()
    per_sub = 2 * L * C
    sub = 0
    for ci, c0 in enumerate(range(0, T, chunk)):
        c1 = min(c0 + chunk, T)
        cdf = oracle.calculate_cdf(sym[:, c0:c1], max_bins)
        assert np.array_equal(enc.cdf[ci].cpu().numpy().view(np.uint16), cdf), ("tables", ci)
        for s0 in range(c0, c1, 256):
            s1 = min(s0 + 256, c1)
            padded, want_len = oracle.encode_fast_new(cdf, np.ascontiguousarray(sym[:, s0:s1]))
            want = oracle.collect_bytes(padded, want_len)
            assert np.array_equal(lengths[sub], want_len), ("lengths", sub)
            assert np.array_equal(payload[offs[sub * per_sub]:offs[(sub + 1) * per_sub]], want), ("bytes", sub)
            sub += 1
    # and back: the decoder reads the same symbols out of the streams
    out_dt = kv.dtype
    out = codec.decode_encoded(enc, kb.to(DEV), vb.to(DEV), fmt="vllm", out_dtype=out_dt)
    mx = maxima.cpu().view(torch.int16).numpy().view(np.uint16)
    want_k = oracle.dequantize(sym[:L], kb.numpy(), mx[0], dt, dt)
    want_v = oracle.dequantize(sym[L:], vb.numpy(), mx[1], dt, dt)
    got = out.cpu().view(torch.int16).numpy().view(np.uint16).reshape(L, 2, T, C)
    for name, g, w in (("keys", got[:, 0], want_k), ("values", got[:, 1], want_v)):
        nan_w = (w & 0x7FFF) > 0x7F80
        nan_g = (g & 0x7FFF) > 0x7F80
        assert np.array_equal(nan_w, nan_g), name
        assert np.array_equal(g[~nan_w], w[~nan_w]), name
    return enc


@pytest.mark.parametrize("heads,head_size,max_bins", [(1, 64, 32), (1, 128, 32), (4, 128, 96), (2, 128, 32)])
def test_saturated_row_late_in_the_sub_chunk(oracle, heads, head_size, max_bins):
    """64 and 128 channels give blocks of 64 and 128 lanes, 512 channels with tables of 97 entries
    blocks of 128: the saturated rows sit at tokens 130..255 of a sub-chunk, past the first block
    size of token rows, in rows of 16 levels (four-bit symbol words) and of 32 levels."""
    from cachegen_amd import codec
    torch.manual_seed(heads * 1000 + head_size + max_bins)
    L, T = 2, 300
    kv = torch.randn((L, 2, T, heads, head_size), dtype=torch.float32)
    kv[0, 0, 200] *= 1e-39                      # keys of layer 0 (32 levels)
    kv[1, 0, 130:133] *= 1e-39                  # keys of layer 1 (16 levels)
    kv[1, 1, 255] *= 2e-39                      # values of layer 1 (16 levels), last row of the first sub-chunk
    kv[0, 1, 299] *= 1e-39                      # values of layer 0, last row of the short sub-chunk
    kv = kv.to(torch.bfloat16)
    kb = torch.tensor([32.0, 16.0])
    vb = torch.tensor([32.0, 16.0])
    enc = _check_against_oracle_on_clamped_symbols(oracle, codec, kv, kb, vb, 256, max_bins, 1)
    # the saturated rows really use the table's last symbol
    last = enc.cdf[0].to(torch.int32) & 0xFFFF
    assert int((last[..., max_bins] - last[..., max_bins - 1]).max()) > 1


@pytest.mark.parametrize("chunk", [256, 600])
def test_table_shorter_than_a_rows_alphabet(oracle, chunk):
    """max_bins below the bins of some rows (a caller's choice the reference does not refuse:
    encoder.py:265-266 takes the maximum, a direct caller of the kernels may not): symbols past
    the table are coded as its last symbol, also in rows that would otherwise travel four bits a
    symbol, and a table of 8 symbols is never indexed at 14."""
    from cachegen_amd import codec
    torch.manual_seed(chunk)
    L, T, H, D = 3, 600, 2, 128
    kv = torch.randn((L, 2, T, H, D), dtype=torch.float32).to(torch.float16)
    kb = torch.tensor([16.0, 8.0, 32.0])
    vb = torch.tensor([12.0, 16.0, 8.0])
    _check_against_oracle_on_clamped_symbols(oracle, codec, kv, kb, vb, chunk, 8, 0)
