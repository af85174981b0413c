"""Limits and error reporting of the HIP path: streams cut at the buffer size, streams that
outgrow 256 bytes, a payload buffer that is too small.  The reference has no defined
behaviour for the last two (enc_new.cu:323-340 writes past its 256-byte slot); here they
are reported through the status word and nothing is written out of bounds."""
import dataclasses

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _mods():
    from cachegen_amd import codec, torchac_hip
    return codec, torchac_hip


@pytest.mark.parametrize("cap", [1, 7, 64, 130])
def test_entry_point_cuts_streams_at_the_buffer_size(oracle, cap):
    """Full length reported, `cap` bytes stored, nothing past the row touched: the oracle's
    bit_sink does the same (it counts bytes it cannot store)."""
    _, tac = _mods()
    rng = np.random.default_rng(cap)
    nl, nt, nc = 2, 256, 70
    sym = rng.integers(0, 31, size=(nl, nt, nc), dtype=np.uint8)       # ~4.9 bits/symbol: ~157 bytes
    cdf = oracle.calculate_cdf(sym, 32)
    want_pad, want_len = oracle.encode_fast_new(cdf, sym, cap=cap)
    assert want_len.max() > cap
    guard = 5
    big = torch.full((nl, nc, cap + guard), 0xEE, dtype=torch.uint8, device=DEV)
    out = big[:, :, :cap]
    lens = torch.zeros((nl, nc), dtype=torch.int32, device=DEV)
    tac.encode_fast_new(torch.from_numpy(cdf.view(np.int16)).to(DEV),
                        torch.from_numpy(sym).to(DEV).view(torch.int8), out, lens)
    assert np.array_equal(lens.cpu().numpy(), want_len)
    got = big.cpu().numpy()
    stored = np.minimum(want_len, cap)
    mask = np.arange(cap)[None, None, :] < stored[..., None]
    assert np.array_equal(got[:, :, :cap][mask], want_pad[mask])
    assert (got[:, :, cap:] == 0xEE).all()


def _overflowing_kv(T, C=64):
    """One layer; channel 1 carries the row maximum, channel 0 is -max on even tokens and
    -max/3 on odd tokens of the first 256 tokens and +max elsewhere: with one table over
    T = 65280 tokens the two symbols of the first sub-chunk have probability 128/65280
    each, i.e. 9 bits per symbol and 288 bytes for that stream."""
    kv = torch.zeros((1, 2, T, 1, C), dtype=torch.float16)
    kv[..., 1] = 1.0
    kv[..., 0] = 1.0
    kv[:, :, 0:256:2, :, 0] = -1.0
    kv[:, :, 1:256:2, :, 0] = -1.0 / 3.0
    return kv


@pytest.mark.parametrize("flags", [None, 2])       # 2: the tables come from the quantizer's own counters (65280 tokens in one block)
def test_stream_longer_than_256_bytes_is_reported(oracle, flags):
    codec, _ = _mods()
    T = 65280
    kv = _overflowing_kv(T)
    bins = torch.tensor([32.0])
    enc = codec.encode_kv(kv.to(DEV), bins, bins, chunk_tokens=T, _test_flags=flags)
    with pytest.raises(RuntimeError, match="exceeded 256 bytes"):
        enc.check()
    lengths = enc.lengths.cpu().numpy()
    # the oracle's coder on the same symbols gives the uncut length
    flat = kv.reshape(1, 2, T, 64).contiguous().view(torch.int16).numpy().view(np.uint16)
    want = oracle.encode_function(flat, bins.numpy(), bins.numpy())
    assert np.array_equal(enc.cdf[0].cpu().numpy().view(np.uint16), want["cdf"])
    data0, want_first, ntok = want["data_chunks"][0]
    assert ntok == 256 and want_first[0, 0] > 256 and want_first[1, 0] > 256
    assert np.array_equal(lengths[0], want_first)
    # offsets advance by the stored (cut) length and every other stream is intact
    offs = enc.offsets.cpu().numpy()
    stored = np.minimum(lengths, 256)
    assert np.array_equal(np.diff(offs), stored.ravel())
    per_sub = lengths[0].size
    got0 = enc.payload[:offs[per_sub]].cpu().numpy()
    assert np.array_equal(got0, data0)                      # the oracle cuts at 256 bytes as well
    # the last sub-chunk (all streams short) decodes to its symbols
    last = lengths.shape[0] - 1
    data_l, len_l, n_l = want["data_chunks"][last]
    assert np.array_equal(enc.payload[offs[last * per_sub]:offs[(last + 1) * per_sub]].cpu().numpy(), data_l)
    assert np.array_equal(lengths[last], len_l)


def test_payload_buffer_too_small_is_reported():
    codec, _ = _mods()
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(2, 300, 4, 64, seed=5, device=DEV)
    bins = torch.tensor([32.0, 16.0])
    enc = codec.encode_kv(kv, bins, bins, chunk_tokens=256)
    enc.check()
    total = enc.total_bytes()
    want = enc.payload[:total].cpu()

    exact = dataclasses.replace(enc, payload=torch.full((total + 64,), 0xEE, dtype=torch.uint8, device=DEV)[:total],
                                status=torch.zeros(1, dtype=torch.int32, device=DEV))
    codec.encode_kv(kv, bins, bins, chunk_tokens=256, out=exact)
    exact.check()
    assert torch.equal(exact.payload.cpu(), want)

    base = torch.full((total + 64,), 0xEE, dtype=torch.uint8, device=DEV)
    small = dataclasses.replace(enc, payload=base[:total - 1],
                                status=torch.zeros(1, dtype=torch.int32, device=DEV))
    codec.encode_kv(kv, bins, bins, chunk_tokens=256, out=small)
    with pytest.raises(RuntimeError, match="payload buffer too small"):
        small.check()
    assert (base[total - 1:] == 0xEE).all()                 # nothing written past the buffer


@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_high_entropy_streams_match_oracle(oracle, dtype, dt):
    """White-noise KV: about 4 bits per symbol, so a block of 256 streams holds well over
    16 KiB of payload and the compaction works through several tiles; 300 tokens make the
    second sub-chunk short, 5 layers an odd number of rows."""
    codec, _ = _mods()
    torch.manual_seed(3)
    L, T, H, D = 5, 300, 4, 128
    kv = torch.randn((L, 2, T, H, D), dtype=torch.float32).to(dtype)
    kb = torch.tensor([32.0, 32.0, 16.0, 32.0, 16.0])
    vb = torch.tensor([32.0, 16.0, 16.0, 32.0, 32.0])
    enc = codec.encode_kv(kv.to(DEV), kb, vb, chunk_tokens=T)
    enc.check()
    flat = kv.reshape(L, 2, T, H * D).contiguous().view(torch.int16).numpy().view(np.uint16)
    want = oracle.encode_function(flat, kb.numpy(), vb.numpy(), dt)
    assert np.array_equal(enc.cdf[0].cpu().numpy().view(np.uint16), want["cdf"])
    bounds = enc.sub_boundaries()
    assert (bounds[1] - bounds[0]) / (2 * L * H * D / 256) > 20000      # bytes per block of 256 streams
    for g, (data, lengths, ntok) in enumerate(want["data_chunks"]):
        assert np.array_equal(enc.lengths[g].cpu().numpy(), lengths)
        assert np.array_equal(enc.payload[bounds[g]:bounds[g + 1]].cpu().numpy(), data)
    out = codec.decode_encoded(enc, kb, vb, out_dtype=dtype)
    _, ref = oracle.decode_function(want, kb.numpy(), vb.numpy(), dt, dt)
    got = out.cpu().reshape(L, 2, T, H * D).contiguous().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, ref)


def test_nan_and_infinite_rows_match_oracle(oracle):
    """Rows whose maximum is infinite or NaN take the decoder's careful path; every other
    row of the same tensor takes the fast one."""
    codec, _ = _mods()
    torch.manual_seed(4)
    L, T, H, D = 2, 64, 2, 64
    kv = torch.randn((L, 2, T, H, D), dtype=torch.float32)
    kv[0, 0, 3, 0, 5] = float("inf")
    kv[1, 1, 9, 1, 7] = float("nan")
    kv[0, 1, 11, 0, 0] = float("-inf")
    kv[1, 0, 20] = 0.0                                   # an all-zero row: 0 * inf
    bins = torch.tensor([32.0, 16.0])
    for dtype, dt in ((torch.float16, 0), (torch.bfloat16, 1)):
        x = kv.to(dtype)
        enc = codec.encode_kv(x.to(DEV), bins, bins, chunk_tokens=T)
        enc.check()
        flat = x.reshape(L, 2, T, H * D).contiguous().view(torch.int16).numpy().view(np.uint16)
        want = oracle.encode_function(flat, bins.numpy(), bins.numpy(), dt)
        assert np.array_equal(enc.payload[:enc.total_bytes()].cpu().numpy(), want["data_chunks"][0][0])
        for out_dtype, odt in ((torch.float16, 0), (torch.bfloat16, 1)):
            out = codec.decode_encoded(enc, bins, bins, out_dtype=out_dtype)
            _, ref = oracle.decode_function(want, bins.numpy(), bins.numpy(), dt, odt)
            got = out.cpu().reshape(L, 2, T, H * D).contiguous().view(torch.int16).numpy().view(np.uint16)
            # 0 * inf has no defined sign or payload (x86 gives the negative default NaN, the GPU
            # the positive one): NaNs must be in the same places, every other value bit-equal
            inf_bits = 0x7C00 if odt == 0 else 0x7F80
            nan_got, nan_ref = (got & 0x7FFF) > inf_bits, (ref & 0x7FFF) > inf_bits
            assert np.array_equal(nan_got, nan_ref), (dtype, out_dtype)
            assert nan_ref.any() and np.array_equal(got[~nan_ref], ref[~nan_ref]), (dtype, out_dtype)


@pytest.mark.parametrize("n", [1, 7, 2048, 2049, 6151, 16383, 16384, 16385, 40000, 300001])
def test_running_sum_of_lengths_at_the_boundaries_of_its_three_forms(n):
    """cg_scan_lengths runs as one block (up to 2048 values), as one block of 1024 threads (up
    to 16384) or as three launches; sums are int64 and negative lengths count as zero."""
    codec, _ = _mods()
    g = torch.Generator().manual_seed(n)
    lengths = torch.randint(0, 257, (n,), generator=g, dtype=torch.int32)
    if n > 10:
        lengths[3] = -5                                   # never produced by the encoder; counted as 0
        lengths[n // 2] = 2_000_000_000                   # sums pass 2^31
        lengths[n - 1] = 2_000_000_000
    want = np.concatenate([[0], np.cumsum(np.maximum(lengths.numpy().astype(np.int64), 0))])
    got = codec.scan_lengths(lengths.to(DEV))
    assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), want)


def test_ties_round_to_even_in_the_fused_quantizer(oracle):
    """Rows made of halves and quarters of the row maximum, so that x * (MAX / max) + MAX lands
    exactly on .5 for many elements (0.5 * 15 + 15 = 22.5 -> 22, -0.5 * 7 + 7 = 3.5 -> 4, ...):
    the fused path rounds inside its packed float-to-byte conversion and must still round half
    to even like torch.round (encoder.py:56-57)."""
    codec, _ = _mods()
    L, T, H, D = 3, 64, 2, 64
    g = torch.Generator().manual_seed(23)
    choices = torch.tensor([1.0, -1.0, 0.5, -0.5, 0.0, 0.25, -0.25, 0.75, -0.75, 0.125])
    kv = choices[torch.randint(0, len(choices), (L, 2, T, H, D), generator=g)]
    kv[..., 0] = 1.0                                             # every row's maximum is exactly 1
    kv[1] *= 2.0                                                 # and exactly 2 in layer 1
    kb = torch.tensor([32.0, 16.0, 12.0])
    vb = torch.tensor([12.0, 32.0, 16.0])
    for dtype, dt in ((torch.float16, 0), (torch.bfloat16, 1)):
        x = kv.to(dtype)
        flat = x.reshape(L, 2, T, H * D).contiguous().view(torch.int16).numpy().view(np.uint16)
        want = oracle.encode_function(flat, kb.numpy(), vb.numpy(), dt)
        wk, _ = oracle.quantize(flat[:, 0], kb.numpy(), dt)
        assert int((wk[0] == 22).sum()) > 0 and int((wk[1] == 4).sum()) > 0      # the ties are there
        enc = codec.encode_kv(x.to(DEV), kb, vb, chunk_tokens=T)
        enc.check()
        assert np.array_equal(enc.cdf[0].cpu().numpy().view(np.uint16), want["cdf"])
        assert np.array_equal(enc.payload[:enc.total_bytes()].cpu().numpy(), want["data_chunks"][0][0])
        lv = codec.encode_kv_levels(x.to(DEV), [(kb, vb), (vb, kb)], chunk_tokens=T)
        assert torch.equal(lv[0].payload[:lv[0].total_bytes()], enc.payload[:enc.total_bytes()])
        want2 = oracle.encode_function(flat, vb.numpy(), kb.numpy(), dt)
        assert np.array_equal(lv[1].payload[:lv[1].total_bytes()].cpu().numpy(), want2["data_chunks"][0][0])


def test_rows_with_several_different_nans_keep_the_largest_pattern(oracle):
    """Two or three NaNs with different payloads and signs in one row: the stored row maximum
    is the largest sign-stripped bit pattern in the fused path, in the plain quantiser and in
    the oracle alike."""
    codec, _ = _mods()
    L, T, H, D = 1, 8, 2, 64
    for dtype, dt, pats in ((torch.float16, 0, [0x7E01, 0xFE55, 0x7C01]), (torch.bfloat16, 1, [0x7FC1, 0xFFD5, 0x7F81])):
        g = torch.Generator().manual_seed(17)
        raw = torch.randn((L, 2, T, H * D), generator=g).to(dtype).view(torch.int16).numpy().view(np.uint16).copy()
        raw[0, 0, 2, 100], raw[0, 0, 2, 3], raw[0, 0, 2, 77] = pats            # the largest one in the middle
        raw[0, 1, 5, 9], raw[0, 1, 5, 120] = pats[2], pats[0]
        x = torch.from_numpy(raw.view(np.int16)).view(dtype).reshape(L, 2, T, H, D)
        bins = torch.tensor([32.0])
        enc = codec.encode_kv(x.to(DEV), bins, bins, chunk_tokens=T)
        enc.check()
        want = oracle.encode_function(raw, bins.numpy(), bins.numpy(), dt)
        got_max = enc.maxima.cpu().view(torch.int16).numpy().view(np.uint16)
        assert got_max[0, 0, 2] == (pats[1] & 0x7FFF) and got_max[1, 0, 5] == pats[0]
        assert np.array_equal(got_max[0], want["max_tensors_key"]) and np.array_equal(got_max[1], want["max_tensors_value"])
        assert np.array_equal(enc.cdf[0].cpu().numpy().view(np.uint16), want["cdf"])
        assert np.array_equal(enc.payload[:enc.total_bytes()].cpu().numpy(), want["data_chunks"][0][0])
        sym, maxima = codec.quantize_kv(x.to(DEV), bins.to(DEV), bins.to(DEV))
        assert np.array_equal(maxima.cpu().view(torch.int16).numpy().view(np.uint16), got_max)


@pytest.mark.parametrize("nt", [1, 2, 7])
def test_streams_that_begin_in_the_last_word_of_an_exact_size_buffer(oracle, nt):
    """The byte buffer ends with the last stream, and that stream is so short that it starts
    inside the buffer's last 32-bit word."""
    _, tac = _mods()
    rng = np.random.default_rng(nt)
    nl, nc = 3, 5
    sym = rng.integers(0, 3, size=(nl, nt, nc), dtype=np.uint8)           # cheap symbols: 1-2 byte streams
    table = np.tile(rng.integers(0, 3, size=(nl, 300, nc), dtype=np.uint8), (1, 1, 1))
    cdf = oracle.calculate_cdf(table, 32)
    pad, lens = oracle.encode_fast_new(cdf, sym)
    data = oracle.collect_bytes(pad, lens)
    assert lens.max() <= 3 and data.size == lens.sum()
    prefix = lens.astype(np.int64).ravel().cumsum().reshape(lens.shape)
    for shift in range(4):                                                 # every alignment of the buffer
        base = torch.zeros(data.size + shift, dtype=torch.uint8, device=DEV)
        base[shift:] = torch.from_numpy(data).to(DEV)
        out = torch.full((nl, nt, nc), 0xEE, dtype=torch.uint8, device=DEV)
        tac.decode_fast_prefsum(torch.from_numpy(cdf.view(np.int16)).to(DEV), base[shift:],
                                torch.from_numpy(prefix).to(DEV), out)
        assert np.array_equal(out.cpu().numpy(), sym), shift


def test_streams_with_bogus_offsets_do_not_disturb_their_neighbours():
    """Offsets that are not running sums of the lengths (negative, beyond the payload, beyond
    4 GiB, or simply another stream's) make their own streams decode to garbage; every other
    stream, including those in the same wavefront, still decodes as before, and nothing is
    read outside the payload (the kernel reads it through a range-checked descriptor)."""
    codec, _ = _mods()
    L, T, H, D = 2, 256, 2, 64
    C = H * D
    g = torch.Generator().manual_seed(5)
    kv = (torch.randn(L, 2, T, H, D, generator=g) * torch.rand(C, generator=g).reshape(H, D)).to(torch.float16).to(DEV)
    bins = torch.tensor([32.0, 16.0])
    enc = codec.encode_kv(kv, bins, bins, chunk_tokens=256)
    clean = codec.decode_encoded(enc, bins, bins, out_dtype=torch.float16)
    nstreams = 2 * L * C
    total = int(enc.offsets[-1])
    rng = np.random.default_rng(11)
    bad = np.unique(np.concatenate([[0, 64, 65, 127, 128, nstreams - 1], rng.integers(0, nstreams, 40)]))
    bogus = np.concatenate([[-5, -10 ** 12, 10 ** 12, (1 << 32) + 7, total + 100, total, total - 1],
                            rng.integers(0, total, bad.size)])[:bad.size]
    offsets = enc.offsets.clone()
    offsets[torch.from_numpy(bad).to(DEV)] = torch.from_numpy(bogus.astype(np.int64)).to(DEV)
    out = codec.decode_kv(enc.cdf, enc.maxima, offsets, enc.payload[:total].clone(), bins, bins, L, T, H, D, 256,
                          out_dtype=torch.float16)
    torch.cuda.synchronize()
    keep = torch.ones(nstreams, dtype=torch.bool)
    keep[torch.from_numpy(bad)] = False
    # stream (row = kv * L + l, channel) is out[l, kv, :, channel]
    got = out.reshape(L, 2, T, C).permute(1, 0, 3, 2).reshape(nstreams, T).cpu()
    want = clean.reshape(L, 2, T, C).permute(1, 0, 3, 2).reshape(nstreams, T).cpu()
    assert torch.equal(got[keep].view(torch.int16), want[keep].view(torch.int16))


def _carry_cases():
    """(table, symbols) pairs whose output runs 0111...1 over one or more whole words (hundreds
    of pending bits in the reference's terms) and is then pushed over the edge by a carry, or
    not, by the symbols that follow."""
    cases = []
    for width in (1, 2, 5):
        cdf = [0, 1, 65535 - width, 65535]                  # the last symbol is tiny and at the very top
        for n in (3, 10, 40):
            for tail in ([], [1], [2, 1], [1, 1, 2], [0]):
                cases.append((cdf, [2] * n + tail))
    cdf = [0, 32767, 32768, 65535]                          # the middle symbol sits just below one half
    for n in (1, 2, 5, 17, 31, 32, 33, 39):
        for last in (0, 1, 2):
            cases.append((cdf, [0] + [1] * n + [last, 2, 0, 1]))
    cdf = [0, 32767, 32769, 65535]                          # the middle symbol straddles one half: every
    for n in (1, 2, 3, 5, 8, 20):                           # repeat adds about fifteen undecided bits
        for last in (0, 1, 2):
            cases.append((cdf, [1] * n + [last, 0, 2]))
    return cases


@pytest.mark.gpu
def test_carries_through_whole_words_of_ones_match_oracle(oracle):
    """The encoder keeps the last complete word back until it knows whether a carry reaches it and
    counts words of all ones behind it: streams that take those paths, through the reference's
    entry point and byte for byte against the oracle's bit-serial pending count."""
    from cachegen_amd import torchac_hip as tac
    cases = _carry_cases()
    nt = max(len(s) for _, s in cases)
    nc = len(cases)
    # every stream is padded with the wide symbol of its own table to the common length
    sym = np.zeros((1, nt, nc), dtype=np.uint8)
    cdf = np.zeros((1, nc, 4), dtype=np.uint16)
    want = []
    for c, (table, symbols) in enumerate(cases):
        wide = max(range(3), key=lambda s: (table + [65536])[s + 1] - table[s])
        padded = symbols + [wide] * (nt - len(symbols))
        sym[0, :, c] = padded
        cdf[0, c] = table
        data, n = oracle.encode_stream(table, padded)
        assert n <= 256
        want.append(bytes(data))
    assert any(b"\xff\xff\xff\xff" in w for w in want) and any(b"\x00\x00\x00\x00" in w for w in want)
    out = torch.zeros((1, nc, 256), dtype=torch.uint8, device=DEV)
    lengths = torch.zeros((1, nc), dtype=torch.int32, device=DEV)
    tac.encode_fast_new(torch.from_numpy(cdf.view(np.int16)).to(DEV), torch.from_numpy(sym.view(np.int8)).to(DEV), out, lengths)
    got_len = lengths.cpu().numpy()[0]
    got = out.cpu().numpy()[0]
    for c, w in enumerate(want):
        assert got_len[c] == len(w), (c, cases[c])
        assert bytes(got[c, :len(w)]) == w, (c, cases[c])
    # and back
    dec = torch.zeros((1, nt, nc), dtype=torch.uint8, device=DEV)
    tac.decode_fast_new(torch.from_numpy(cdf.view(np.int16)).to(DEV), out, lengths, dec)
    assert np.array_equal(dec.cpu().numpy(), sym)


@pytest.mark.gpu
@pytest.mark.parametrize("chunk", [256, 300])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_four_bit_symbol_words_give_the_same_streams_as_byte_words(dtype, chunk):
    """Rows of at most 15 symbols cross from the quantizer to the coder four bits a symbol.  The
    other form (a byte a symbol, the library's test entry point) must give the same tables, streams and maxima,
    also for token rows whose scale overflows (bfloat16 maxima below 2^-125: MAX / max is
    infinite, every non-zero value saturates to the table's last symbol) and rows of zeros."""
    codec, _ = _mods()
    torch.manual_seed(11)
    L, T, H, D = 3, 300, 4, 128
    kv = torch.randn((L, 2, T, H, D), dtype=torch.float32)
    kv[1, 0, 7] = 0.0                                       # a row of zeros
    if dtype == torch.bfloat16:
        kv[2, 1, 40:44] *= 1e-39                            # denormal maxima: the scale overflows
        kv[0, 0, 299] *= 3e-39
        kv[1, 1, 100] *= 1e-39
    kv = kv.to(dtype).to(DEV)
    kb = torch.tensor([32.0, 16.0, 12.0])
    vb = torch.tensor([16.0, 8.0, 16.0])
    got = codec.encode_kv(kv, kb, vb, chunk_tokens=chunk)
    got.check()
    ref = codec.encode_kv(kv, kb, vb, chunk_tokens=chunk, _test_flags=1)          # CG_TEST_BYTE_SYMBOLS
    ref.check()
    n = ref.total_bytes()
    assert got.total_bytes() == n
    assert torch.equal(got.cdf, ref.cdf) and torch.equal(got.lengths, ref.lengths) and torch.equal(got.offsets, ref.offsets)
    assert torch.equal(got.payload[:n], ref.payload[:n]) and torch.equal(got.maxima, ref.maxima)
    if dtype == torch.bfloat16:
        # the saturated rows really use the last table symbol (value layer 2 has 16 levels: symbol 31 of 33 entries)
        last = ref.cdf[0, 3 + 2].to(torch.int32) & 0xFFFF   # row = L + layer 2
        assert int((last[:, 32] - last[:, 31]).max()) > 1
    # the decoder gives the coder's symbols back: every value within half a step of its row's scale
    out = codec.decode_encoded(got, kb, vb, out_dtype=dtype).float().cpu()
    src = kv.float().cpu()
    mx = src.abs().amax(dim=(-1, -2), keepdim=True)
    step = mx / (torch.floor(torch.cat([kb, vb]).view(2, L).t().reshape(L, 2, 1, 1, 1) / 2) - 1)
    ok = (out - src).abs() <= 0.6 * step + 1e-30             # half a step and the 16-bit rounding of the output
    sane = mx > 1e-30                                       # rows whose scale did not overflow
    assert bool((ok | ~sane.expand_as(ok)).all())


def test_more_than_65535_rows_are_refused_and_65535_are_coded(oracle):
    """The stream kernels run on a grid of (channel tile, row, sub-chunk): a call with more rows
    than a grid dimension holds is refused before anything is launched, and the largest number
    of rows that fits is coded like any other."""
    import cachegen_amd.torchac_hip as tac
    g = torch.Generator().manual_seed(7)
    cdf_row = torch.tensor([0, 21845, 65535], dtype=torch.int32).to(torch.int16)
    for nl, ok in ((65536, False), (65535, True)):
        cdf = cdf_row.expand(nl, 1, 3).contiguous().to(DEV)
        sym = torch.randint(0, 2, (nl, 5, 1), generator=g, dtype=torch.int8).to(DEV)
        buf = torch.zeros((nl, 1, 16), dtype=torch.uint8, device=DEV)
        lengths = torch.zeros((nl, 1), dtype=torch.int32, device=DEV)
        if not ok:
            with pytest.raises(RuntimeError, match="at most 65535"):
                tac.encode_fast_new(cdf, sym, buf, lengths)
            continue
        tac.encode_fast_new(cdf, sym, buf, lengths)
        out = torch.zeros((nl, 5, 1), dtype=torch.uint8, device=DEV)
        tac.decode_fast_new(cdf, buf, lengths, out)
        assert torch.equal(out.cpu(), sym.cpu().to(torch.uint8))
        # a few rows against the oracle, the last one among them
        for r in (0, 1, 40000, nl - 1):
            want, n = oracle.encode_stream(cdf_row.numpy().view(np.uint16), sym[r, :, 0].cpu().numpy().astype(np.uint8))
            assert int(lengths[r, 0]) == n
            assert buf[r, 0, :n].cpu().numpy().tobytes() == want, r
