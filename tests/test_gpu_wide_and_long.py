"""Wide rows (2048 and 4096 channels: the Llama-2-7B shape of 32 heads x 128) and long
contexts (16 384 tokens of that shape; 32 768 tokens of the 70B shape in 1500-token chunks).

Small slices of those shapes go through the oracle bit for bit; the full-size runs are
checked through properties that do not depend on size (re-encoding the decoded cache gives
the same bytes, a chunk encoded alone equals its slice of the batch, the fused decoder
agrees with the entry-point path followed by tensor-op dequantisation, table invariants,
reconstruction within half a quantisation step), and one chunk of each is pulled back to
the host and compared with the oracle bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _bins(model):
    from cachegen_amd.serde import cachegen_basics as B
    cfg = B.CacheGenConfig.from_model_name(model)
    return B.make_key_bins(cfg).to(DEV), B.make_value_bins(cfg).to(DEV)


def _compare_chunk_with_oracle(oracle, enc, bounds, i, flat_chunk, kb, vb, dt, got_chunk, odt, label):
    """Chunk i of `enc` and its decoded 16-bit values against the oracle run on the chunk's
    input bits `flat_chunk` [L, 2, n, C]."""
    want = oracle.encode_function(flat_chunk, kb, vb, dt)
    cdf, max_k, max_v, subs = enc.chunk(i, bounds)
    assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"]), label
    assert np.array_equal(bits(max_k)[..., 0], want["max_tensors_key"]), label
    assert np.array_equal(bits(max_v)[..., 0], want["max_tensors_value"]), label
    assert len(subs) == len(want["data_chunks"]), label
    for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
        assert n == wn and np.array_equal(l.cpu().numpy(), wl), label
        assert np.array_equal(b.cpu().numpy(), wb), label
    _, want_kv = oracle.decode_function(want, kb, vb, max_dt=dt, out_dt=odt)
    assert np.array_equal(got_chunk, want_kv), label


# --------------------------------------------------------------------------- #
# slices of the wide shapes against the oracle
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("H", [16, 32])
@pytest.mark.parametrize("chunk", [256, 300])
def test_wide_rows_match_oracle(oracle, dtype, dt, fmt, H, chunk):
    """C = 2048 and 4096: four and eight 128-bit loads per lane and token row in the fused
    quantiser, eight and sixteen channel tiles per row in the coders."""
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    L, T, D = 2, 300, 128
    C = H * D
    kv = make_kv(L, T, H, D, seed=400 + H + chunk, dtype=dtype)
    kv[1, 0, 7] = 0                                                  # an all-zero row
    kb = np.array([32.0, 16.0], dtype=np.float32)
    vb = np.array([16.0, 32.0], dtype=np.float32)
    label = dict(H=H, chunk=chunk, fmt=fmt, dtype=str(dtype))
    print(label, flush=True)
    dev_kv = kv.to(DEV)
    src = dev_kv.permute(0, 1, 3, 2, 4).contiguous() if fmt == "huggingface" else dev_kv
    enc = codec.encode_kv(src, torch.from_numpy(kb), torch.from_numpy(vb), chunk_tokens=chunk, fmt=fmt)
    enc.check()
    out = codec.decode_encoded(enc, torch.from_numpy(kb), torch.from_numpy(vb), fmt=fmt, out_dtype=dtype)
    got = out if fmt == "vllm" else out.permute(0, 1, 3, 2, 4)
    got = bits(got).reshape(L, 2, T, C)
    flat = bits(kv).reshape(L, 2, T, C)
    bounds = enc.sub_boundaries()
    for i, t0 in enumerate(range(0, T, chunk)):
        t1 = min(t0 + chunk, T)
        _compare_chunk_with_oracle(oracle, enc, bounds, i, flat[:, :, t0:t1], kb, vb, dt, got[:, :, t0:t1], dt, label)
    # the plain quantiser at these widths
    sym, maxima = codec.quantize_kv(src, torch.from_numpy(kb).to(DEV), torch.from_numpy(vb).to(DEV), fmt=fmt)
    want_k, max_k = oracle.quantize(flat[:, 0], kb, dt)
    want_v, max_v = oracle.quantize(flat[:, 1], vb, dt)
    assert np.array_equal(sym.cpu().numpy(), np.concatenate([want_k, want_v]))
    assert np.array_equal(bits(maxima), np.stack([max_k, max_v]))


# --------------------------------------------------------------------------- #
# full-size properties
# --------------------------------------------------------------------------- #
def _half_step_ok(kv, out, kb, vb, group):
    L, _, T, H, D = kv.shape
    maxq = torch.stack([kb, vb], dim=1).div(2, rounding_mode="floor").sub(1)[:, :, None, None]
    for l0 in range(0, L, group):
        x = kv[l0:l0 + group].reshape(-1, 2, T, H * D).float()
        y = out[l0:l0 + group].reshape(-1, 2, T, H * D).float()
        step = x.abs().amax(dim=-1, keepdim=True) / maxq[l0:l0 + group]
        ok = bool(((x - y).abs() <= 0.52 * step).all())
        del x, y, step
        if not ok:
            return False
    return True


def _tables_and_lengths_ok(enc):
    for c in range(enc.cdf.shape[0]):                   # per chunk to bound memory
        cdf = enc.cdf[c].view(torch.uint16).to(torch.int32)
        assert int(cdf[..., 0].max()) == 0 and int(cdf[..., -1].min()) == 65535
        assert bool((cdf[..., 1:] > cdf[..., :-1]).all())
        del cdf
    assert int(enc.lengths.min()) >= 1 and int(enc.lengths.max()) <= 256
    off = enc.offsets
    assert int(off[0]) == 0 and bool((off[1:] - off[:-1] == enc.lengths.flatten()).all())
    assert enc.total_bytes() == int(enc.lengths.sum(dtype=torch.int64))


@pytest.fixture(scope="module")
def llama7b_16k():
    """32 layers x {K,V} x 16 384 tokens x 32 heads x 128, fp16 (8.6 GB), table per 256 tokens;
    more than 2^32 symbols, so stream and element indices need 64 bits."""
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    print("generating 32 x 2 x 16384 x 4096", flush=True)
    kv = make_kv(32, 16384, 32, 128, seed=1237, device=DEV)
    kb, vb = _bins("lmsys/longchat-7b-16k")
    print("encoding", flush=True)
    enc = codec.encode_kv(kv, kb, vb, chunk_tokens=256)
    enc.check()
    out = codec.decode_encoded(enc, kb, vb, fmt="vllm", out_dtype=torch.float16)
    torch.cuda.synchronize()
    yield kv, kb, vb, enc, out
    del kv, enc, out
    torch.cuda.empty_cache()


def test_llama7b_16k_round_trip_and_tables(llama7b_16k):
    kv, kb, vb, enc, out = llama7b_16k
    assert enc.lengths.numel() == 64 * 64 * 4096 and enc.cdf.shape[0] == 64
    assert _half_step_ok(kv, out, kb, vb, 4)
    _tables_and_lengths_ok(enc)
    L, _, T, H, D = kv.shape
    for l0 in range(0, L, 8):
        assert torch.equal(enc.maxima[:, l0:l0 + 8],
                           kv[l0:l0 + 8].reshape(8, 2, T, H * D).abs().amax(dim=-1).permute(1, 0, 2))


def test_llama7b_16k_reencoding_is_idempotent(llama7b_16k):
    from cachegen_amd import codec
    kv, kb, vb, enc, out = llama7b_16k
    again = codec.encode_kv(out, kb, vb, chunk_tokens=256)
    again.check()
    n = enc.total_bytes()
    assert again.total_bytes() == n
    assert torch.equal(again.lengths, enc.lengths)
    assert torch.equal(again.cdf, enc.cdf)
    assert torch.equal(again.payload[:n], enc.payload[:n])


def test_llama7b_16k_chunks_are_independent_and_match_oracle(oracle, llama7b_16k):
    """Chunks from both ends and the middle (the last one lies past 2^32 symbols) encoded alone
    equal their slices of the batch; one of them goes through the oracle bit for bit."""
    from cachegen_amd import codec
    kv, kb, vb, enc, out = llama7b_16k
    bounds = enc.sub_boundaries()
    for k in (0, 37, 63):
        one = codec.encode_kv(kv[:, :, k * 256:(k + 1) * 256], kb, vb, chunk_tokens=256)
        one.check()
        cdf, mk, mv, subs = enc.chunk(k, bounds)
        assert torch.equal(one.cdf[0], cdf)
        assert torch.equal(one.lengths[0], subs[0][1])
        assert torch.equal(one.payload[:one.total_bytes()], subs[0][0])
        assert torch.equal(one.maxima[0, :, :, None], mk)
    k = 63
    flat = bits(kv[:, :, k * 256:(k + 1) * 256]).reshape(32, 2, 256, 4096)
    got = bits(out[:, :, k * 256:(k + 1) * 256]).reshape(32, 2, 256, 4096)
    _compare_chunk_with_oracle(oracle, enc, bounds, k, flat, kb.cpu().numpy(), vb.cpu().numpy(), 0, got, 0,
                               "16k-token cache, chunk 63")


def test_llama7b_16k_fused_decode_agrees_with_entry_points(llama7b_16k):
    from cachegen_amd import codec, torchac_hip as tac
    from cachegen_amd.serde.cachegen_decoder import do_dequantize
    kv, kb, vb, enc, out = llama7b_16k
    bounds = enc.sub_boundaries()
    k = 41
    cdf, mk, mv, subs = enc.chunk(k, bounds)
    data, lengths, n = subs[0]
    prefix = codec.scan_lengths(lengths)[1:].view(lengths.shape)
    sym = torch.zeros((64, n, 4096), dtype=torch.uint8, device=DEV)
    tac.decode_fast_prefsum(cdf, data, prefix, sym)
    key = do_dequantize(sym[:32].float(), kb, mk).to(torch.float16)
    val = do_dequantize(sym[32:].float(), vb, mv).to(torch.float16)
    got = out[:, :, k * 256:(k + 1) * 256].reshape(32, 2, n, 4096)
    assert torch.equal(got[:, 0], key) and torch.equal(got[:, 1], val)
    qsym, _ = codec.quantize_kv(kv[:, :, k * 256:(k + 1) * 256], kb, vb)
    assert torch.equal(qsym, sym)


@pytest.fixture(scope="module")
def llama70b_32k():
    """80 layers x {K,V} x 32 768 tokens x 8 heads x 128, fp16 (10.7 GB), 1500-token chunks
    (21 of them and one of 1268 tokens), each cut into streams of 5 x 256 + 220 tokens."""
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    print("generating 80 x 2 x 32768 x 1024", flush=True)
    kv = make_kv(80, 32768, 8, 128, seed=1238, device=DEV)
    kb, vb = _bins("Yukang/LongAlpaca-70B-16k")
    print("encoding", flush=True)
    enc = codec.encode_kv(kv, kb, vb, chunk_tokens=1500)
    enc.check()
    out = codec.decode_encoded(enc, kb, vb, fmt="vllm", out_dtype=torch.float16)
    torch.cuda.synchronize()
    yield kv, kb, vb, enc, out
    del kv, enc, out
    torch.cuda.empty_cache()


def test_llama70b_32k_round_trip_and_tables(llama70b_32k):
    kv, kb, vb, enc, out = llama70b_32k
    assert enc.cdf.shape[0] == 22 and enc.lengths.shape[0] == 21 * 6 + 5
    assert _half_step_ok(kv, out, kb, vb, 8)
    _tables_and_lengths_ok(enc)


def test_llama70b_32k_reencoding_is_idempotent(llama70b_32k):
    from cachegen_amd import codec
    kv, kb, vb, enc, out = llama70b_32k
    again = codec.encode_kv(out, kb, vb, chunk_tokens=1500)
    again.check()
    n = enc.total_bytes()
    assert again.total_bytes() == n
    assert torch.equal(again.lengths, enc.lengths)
    assert torch.equal(again.cdf, enc.cdf)
    assert torch.equal(again.payload[:n], enc.payload[:n])


def test_llama70b_32k_chunks_are_independent_and_match_oracle(oracle, llama70b_32k):
    """The first, a middle and the ragged last chunk encoded alone equal their slices of the
    batch; the last one (1268 tokens = 4 x 256 + 244) goes through the oracle bit for bit."""
    from cachegen_amd import codec
    kv, kb, vb, enc, out = llama70b_32k
    T = kv.shape[2]
    bounds = enc.sub_boundaries()
    for k in (0, 11, 21):
        t0, t1 = k * 1500, min((k + 1) * 1500, T)
        one = codec.encode_kv(kv[:, :, t0:t1], kb, vb, chunk_tokens=1500)
        one.check()
        one_bounds = one.sub_boundaries()
        cdf, mk, mv, subs = enc.chunk(k, bounds)
        assert torch.equal(one.cdf[0], cdf)
        assert torch.equal(one.maxima[0, :, :, None], mk) and torch.equal(one.maxima[1, :, :, None], mv)
        _, _, _, one_subs = one.chunk(0, one_bounds)
        assert len(one_subs) == len(subs)
        for (b, l, n), (ob, ol, on) in zip(subs, one_subs):
            assert n == on and torch.equal(l, ol) and torch.equal(b, ob)
    k = 21
    t0 = k * 1500
    flat = bits(kv[:, :, t0:T]).reshape(80, 2, T - t0, 1024)
    got = bits(out[:, :, t0:T]).reshape(80, 2, T - t0, 1024)
    _compare_chunk_with_oracle(oracle, enc, bounds, k, flat, kb.cpu().numpy(), vb.cpu().numpy(), 0, got, 0,
                               "32k-token cache, chunk 21")


def test_llama70b_32k_fused_decode_agrees_with_entry_points(llama70b_32k):
    """Sub-chunk 3 of chunk 9: decode_fast_prefsum on its slice of the payload with the chunk's
    tables, then tensor-op dequantisation."""
    from cachegen_amd import codec, torchac_hip as tac
    from cachegen_amd.serde.cachegen_decoder import do_dequantize
    kv, kb, vb, enc, out = llama70b_32k
    bounds = enc.sub_boundaries()
    k, j = 9, 3
    cdf, mk, mv, subs = enc.chunk(k, bounds)
    data, lengths, n = subs[j]
    t0 = k * 1500 + j * 256
    prefix = codec.scan_lengths(lengths)[1:].view(lengths.shape)
    sym = torch.zeros((160, n, 1024), dtype=torch.uint8, device=DEV)
    tac.decode_fast_prefsum(cdf, data, prefix, sym)
    key = do_dequantize(sym[:80].float(), kb, mk[:, j * 256:j * 256 + n]).to(torch.float16)
    val = do_dequantize(sym[80:].float(), vb, mv[:, j * 256:j * 256 + n]).to(torch.float16)
    got = out[:, :, t0:t0 + n].reshape(80, 2, n, 1024)
    assert torch.equal(got[:, 0], key) and torch.equal(got[:, 1], val)
    qsym, _ = codec.quantize_kv(kv[:, :, t0:t0 + n], kb, vb)
    assert torch.equal(qsym, sym)
