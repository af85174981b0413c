"""Parity of the HIP kernels with the CPU oracle, through the C ABI (bit-exact).

Every test runs the product path (cachegen_amd -> lib/libcachegen_hip.so) on the GPU and
the oracle on the same seeded inputs on the CPU, and compares integers / bit patterns."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def bits(t):
    """16-bit float tensor -> numpy uint16 bit patterns (CPU)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def gpu_mods():
    from cachegen_amd import codec, torchac_hip
    return codec, torchac_hip


def random_symbols(rng, nl, nt, nc, nsym, alpha=0.4):
    p = rng.dirichlet(np.ones(nsym) * alpha, size=(nl, nc))
    u = rng.random((nl, nt, nc))
    cum = np.cumsum(p, axis=-1)[:, None, :, :]
    return (u[..., None] > cum).sum(-1).clip(0, nsym - 1).astype(np.uint8)


# --------------------------------------------------------------------------- #
# quantization
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("shape", [(2, 300, 8, 64), (3, 40, 4, 128), (2, 17, 3, 20), (1, 5, 32, 128)])
def test_quantize_matches_oracle(oracle, dtype, dt, fmt, shape):
    codec, _ = gpu_mods()
    from cachegen_amd.kvgen import make_kv
    L, T, H, D = shape
    kv = make_kv(L, T, H, D, seed=21, dtype=dtype)
    kv[0, 0, 1] = 0                                       # an all-zero row
    kbins = torch.tensor([32.0, 16.0, 12.0][:L] + [16.0] * max(0, L - 3))
    vbins = torch.tensor([16.0, 32.0, 8.0][:L] + [12.0] * max(0, L - 3))
    dev = kv.to(DEV)
    if fmt == "huggingface":
        dev = dev.permute(0, 1, 3, 2, 4).contiguous()     # [L,2,H,T,D] storage
    sym, maxima = codec.quantize_kv(dev, kbins.to(DEV), vbins.to(DEV), fmt=fmt)
    flat = bits(kv).reshape(L, 2, T, H * D)
    want_k, max_k = oracle.quantize(flat[:, 0], kbins.numpy(), dt)
    want_v, max_v = oracle.quantize(flat[:, 1], vbins.numpy(), dt)
    assert np.array_equal(sym.cpu().numpy(), np.concatenate([want_k, want_v]))
    assert np.array_equal(bits(maxima), np.stack([max_k, max_v]))


def test_quantize_known_answer_on_gpu():
    codec, _ = gpu_mods()
    x = torch.tensor([1.0, -1.0, 0.5, 0.0] * 2, dtype=torch.float16).view(1, 1, 1, 1, 8)
    kv = torch.cat([x, x], dim=1).to(DEV)
    sym, maxima = codec.quantize_kv(kv, torch.tensor([32.0], device=DEV), torch.tensor([12.0], device=DEV))
    assert sym[0, 0].tolist() == [30, 0, 22, 15] * 2
    assert sym[1, 0].tolist() == [10, 0, 8, 5] * 2
    assert maxima.flatten().tolist() == [1.0, 1.0]


# --------------------------------------------------------------------------- #
# tables
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("max_bins,nl,nt,nc", [(32, 4, 256, 1024), (32, 2, 1500, 96), (16, 3, 7, 33),
                                               (63, 2, 900, 200), (12, 1, 65535, 8), (100, 2, 300, 70)])
def test_calculate_cdf_matches_oracle(oracle, max_bins, nl, nt, nc):
    _, tac = gpu_mods()
    rng = np.random.default_rng(max_bins + nt)
    sym = random_symbols(rng, nl, nt + 9, nc, max_bins - 1)
    dev = torch.from_numpy(sym).to(DEV).view(torch.int8)
    got = tac.calculate_cdf(dev[:, 4:4 + nt, :], max_bins)            # a strided view
    want = oracle.calculate_cdf(sym[:, 4:4 + nt, :], max_bins)
    assert got.dtype == torch.int16 and tuple(got.shape) == (nl, nc, max_bins + 1)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want)


def test_calculate_cdf_known_answer_on_gpu():
    _, tac = gpu_mods()
    sym = torch.tensor([0, 0, 1, 30], dtype=torch.int8, device=DEV).view(1, 4, 1)
    cdf = tac.calculate_cdf(sym, 32).cpu().numpy().view(np.uint16)[0, 0].tolist()
    assert cdf == [0, 32752] + [49127 + i for i in range(2, 31)] + [65534, 65535]


# --------------------------------------------------------------------------- #
# coder entry points
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("max_bins,nl,nt,nc,table_tokens", [
    (32, 4, 256, 1024, 256), (32, 3, 256, 96, 1500), (16, 2, 44, 33, 300), (32, 2, 1, 64, 1),
    (64, 2, 256, 130, 256), (12, 5, 100, 7, 100),
    # tables of more than 65 entries: the search that is not unrolled; more than 80 entries: blocks of 128 lanes
    (80, 2, 256, 300, 256), (96, 2, 256, 200, 256), (128, 2, 256, 300, 700), (128, 1, 100, 64, 100), (100, 3, 31, 5, 400)])
def test_encode_and_decode_entry_points_match_oracle(oracle, max_bins, nl, nt, nc, table_tokens):
    _, tac = gpu_mods()
    rng = np.random.default_rng(nl * 1000 + nt + nc)
    full = random_symbols(rng, nl, table_tokens, nc, max_bins - 1)
    start = (table_tokens - nt) // 2
    cdf = oracle.calculate_cdf(full, max_bins)
    part = full[:, start:start + nt, :]
    want_pad, want_len = oracle.encode_fast_new(cdf, part)

    d_full = torch.from_numpy(full).to(DEV).view(torch.int8)
    d_cdf = torch.from_numpy(cdf.view(np.int16)).to(DEV)
    out = torch.full((nl, nc, 256), 0xEE, dtype=torch.uint8, device=DEV)
    lens = torch.zeros((nl, nc), dtype=torch.int32, device=DEV)
    tac.encode_fast_new(d_cdf, d_full[:, start:start + nt, :], out, lens)
    got_len = lens.cpu().numpy()
    got_pad = out.cpu().numpy()
    assert np.array_equal(got_len, want_len)
    mask = np.arange(256)[None, None, :] < want_len[..., None]
    assert np.array_equal(got_pad[mask], want_pad[mask])
    assert (got_pad[~mask] == 0xEE).all()                   # bytes past the length untouched

    # decode: concatenated streams + inclusive prefix sums, into a strided view
    data = oracle.collect_bytes(want_pad, want_len)
    prefix = want_len.astype(np.int64).ravel().cumsum().reshape(want_len.shape)
    buf = torch.zeros((nl, nt + 6, nc), dtype=torch.uint8, device=DEV)
    tac.decode_fast_prefsum(d_cdf, torch.from_numpy(data).to(DEV), torch.from_numpy(prefix).to(DEV),
                            buf[:, 3:3 + nt, :])
    assert np.array_equal(buf[:, 3:3 + nt, :].cpu().numpy(), part)
    assert int(buf[:, :3].max()) == 0 and int(buf[:, 3 + nt:].max()) == 0
    # decode from the padded buffer
    buf2 = torch.zeros((nl, nt, nc), dtype=torch.uint8, device=DEV)
    tac.decode_fast_new(d_cdf, out, lens, buf2)
    assert np.array_equal(buf2.cpu().numpy(), part)


def test_coder_known_answers_on_gpu():
    _, tac = gpu_mods()
    cdf3 = torch.tensor([0, 16384, 49152 - 65536, -1], dtype=torch.int16, device=DEV).view(1, 1, 4)
    cases = [([1, 0], [0x48]), ([1, 2], [0xA8]), ([1] * 40, list(int("0" + "1" * 41 + "000000", 2).to_bytes(6, "big")))]
    for syms, want in cases:
        s = torch.tensor(syms, dtype=torch.int8, device=DEV).view(1, -1, 1)
        out = torch.zeros((1, 1, 256), dtype=torch.uint8, device=DEV)
        lens = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
        tac.encode_fast_new(cdf3, s, out, lens)
        assert int(lens) == len(want) and out[0, 0, :len(want)].tolist() == want
        back = torch.zeros((1, len(syms), 1), dtype=torch.uint8, device=DEV)
        tac.decode_fast_new(cdf3, out, lens, back)
        assert back.flatten().tolist() == syms


def test_unaligned_output_buffer_and_odd_channels(oracle):
    _, tac = gpu_mods()
    rng = np.random.default_rng(77)
    nl, nt, nc = 2, 200, 13
    sym = random_symbols(rng, nl, nt, nc, 31)
    cdf = oracle.calculate_cdf(sym, 32)
    want_pad, want_len = oracle.encode_fast_new(cdf, sym, cap=255)
    big = torch.zeros(nl * nc * 255 + 1, dtype=torch.uint8, device=DEV)
    out = big[1:].view(nl, nc, 255)                          # odd base address, odd row length
    lens = torch.zeros((nl, nc), dtype=torch.int32, device=DEV)
    tac.encode_fast_new(torch.from_numpy(cdf.view(np.int16)).to(DEV),
                        torch.from_numpy(sym).to(DEV).view(torch.int8), out, lens)
    assert np.array_equal(lens.cpu().numpy(), want_len)
    mask = np.arange(255)[None, None, :] < want_len[..., None]
    assert np.array_equal(out.cpu().numpy()[mask], want_pad[mask])
    back = torch.zeros((nl, nt, nc), dtype=torch.uint8, device=DEV)
    tac.decode_fast_new(torch.from_numpy(cdf.view(np.int16)).to(DEV), out, lens, back)
    assert np.array_equal(back.cpu().numpy(), sym)


def test_entry_point_errors():
    _, tac = gpu_mods()
    cdf = torch.zeros((2, 64, 33), dtype=torch.int16, device=DEV)
    sym = torch.zeros((2, 257, 64), dtype=torch.int8, device=DEV)
    out = torch.zeros((2, 64, 256), dtype=torch.uint8, device=DEV)
    lens = torch.zeros((2, 64), dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="less than or equal to 256"):
        tac.encode_fast_new(cdf, sym, out, lens)
    with pytest.raises(RuntimeError, match="should be on GPU"):
        tac.encode_fast_new(cdf.cpu(), sym[:, :4], out, lens)
    with pytest.raises(RuntimeError, match="same number of layers"):
        tac.encode_fast_new(cdf[:1], sym[:, :4], out, lens)
    with pytest.raises(RuntimeError, match="Max bins must be less than"):
        tac.calculate_cdf(sym[:, :4], 4096)


# --------------------------------------------------------------------------- #
# fused whole-tensor path
# --------------------------------------------------------------------------- #
def _tables(L):
    k = torch.tensor([32.0] * (L // 2) + [16.0] * (L - L // 2))
    return k, k.clone()


@pytest.mark.parametrize("bins,S", [((128.0, 96.0, 16.0), 256), ((96.0, 70.0, 32.0), 600), ((128.0, 128.0, 128.0), 300)])
def test_fused_path_with_tables_up_to_the_length_limit_matches_oracle(oracle, bins, S):
    """Tables of 97 and 129 entries (CG_MAX_LP) through cg_encode_kv and cg_decode_kv: blocks of
    128 lanes, the search that is not unrolled, rows of 16 levels next to rows of 128."""
    codec, _ = gpu_mods()
    from cachegen_amd.kvgen import make_kv
    L, T, H, D = 3, 600, 3, 64
    kv = make_kv(L, T, H, D, seed=77, dtype=torch.float16)
    kbins = torch.tensor(bins)
    vbins = torch.tensor(bins[::-1])
    enc = codec.encode_kv(kv.to(DEV), kbins.to(DEV), vbins.to(DEV), chunk_tokens=S)
    enc.check()
    assert enc.cdf.shape[-1] == int(max(bins)) + 1
    flat = bits(kv).reshape(L, 2, T, H * D)
    bounds = enc.sub_boundaries()
    sub = 0
    out = codec.decode_encoded(enc, kbins.to(DEV), vbins.to(DEV), fmt="vllm", out_dtype=torch.float16)
    got_kv = bits(out).reshape(L, 2, T, H * D)
    for ci, c0 in enumerate(range(0, T, S)):
        c1 = min(c0 + S, T)
        want = oracle.encode_function(np.ascontiguousarray(flat[:, :, c0:c1]), kbins.numpy(), vbins.numpy(), 0)
        cdf, _, _, subs = enc.chunk(ci, bounds)
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert n == wn and np.array_equal(l.cpu().numpy(), wl) and np.array_equal(b.cpu().numpy(), wb)
            sub += 1
        _, want_kv = oracle.decode_function(want, kbins.numpy(), vbins.numpy())
        assert np.array_equal(got_kv[:, :, c0:c1], want_kv)


@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("L,T,H,D,S", [(2, 512, 8, 64, 512),      # benchmark config 1: two sub-chunks share a table
                                       (2, 512, 8, 64, 256),      # a table per 256 tokens
                                       (2, 300, 4, 32, 300),      # ragged: 256 + 44
                                       (3, 700, 2, 40, 300),      # ragged chunks and sub-chunks, C = 80
                                       (1, 1600, 2, 64, 1500)])   # long chunk: 6 + 1 sub-chunks
def test_fused_encode_decode_match_oracle(oracle, dtype, dt, L, T, H, D, S):
    codec, _ = gpu_mods()
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(L, T, H, D, seed=31 + L + T, dtype=dtype)
    kbins, vbins = _tables(L)
    enc = codec.encode_kv(kv.to(DEV), kbins.to(DEV), vbins.to(DEV), chunk_tokens=S)
    enc.check()
    flat = bits(kv).reshape(L, 2, T, H * D)
    bounds = enc.sub_boundaries()
    C = H * D
    for i, t0 in enumerate(range(0, T, S)):
        t1 = min(t0 + S, T)
        want = oracle.encode_function(flat[:, :, t0:t1], kbins.numpy(), vbins.numpy(), dt)
        cdf, max_k, max_v, subs = enc.chunk(i, bounds)
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"])
        assert np.array_equal(bits(max_k)[..., 0], want["max_tensors_key"])
        assert np.array_equal(bits(max_v)[..., 0], want["max_tensors_value"])
        assert len(subs) == len(want["data_chunks"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert n == wn
            assert np.array_equal(l.cpu().numpy(), wl)
            assert np.array_equal(b.cpu().numpy(), wb)
    for fmt, out_dtype, odt in (("vllm", torch.bfloat16, 1), ("huggingface", torch.float16, 0)):
        out = codec.decode_encoded(enc, kbins.to(DEV), vbins.to(DEV), fmt=fmt)
        assert out.dtype == out_dtype
        assert tuple(out.shape) == ((L, 2, T, H, D) if fmt == "vllm" else (L, 2, H, T, D))
        got = out if fmt == "vllm" else out.permute(0, 1, 3, 2, 4)
        got = bits(got.contiguous()).reshape(L, 2, T, C)
        for i, t0 in enumerate(range(0, T, S)):
            t1 = min(t0 + S, T)
            want = oracle.encode_function(flat[:, :, t0:t1], kbins.numpy(), vbins.numpy(), dt)
            _, want_kv = oracle.decode_function(want, kbins.numpy(), vbins.numpy(), max_dt=dt, out_dt=odt)
            assert np.array_equal(got[:, :, t0:t1], want_kv)


def test_serializer_round_trip_like_reference_tests(oracle, monkeypatch):
    """The three behaviours the reference's own serde test asserts (equal pickle sizes for
    the two layouts, heads/size fields, shape after a round trip with an unmatched size),
    plus value parity of the decoded tensor with the oracle."""
    monkeypatch.setenv("QUANT_LEVEL", "2")
    from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
    from cachegen_amd.serde import CreateSerde
    from cachegen_amd.serde.cachegen_basics import CacheGenEncoderOutput
    torch.manual_seed(5)
    ntok = 236
    cfg = LMCacheEngineConfig.from_defaults(chunk_size=256)
    name = "mistralai/Mistral-7B-Instruct-v0.2"
    kv = torch.rand((32, 2, ntok, 8, 128), dtype=torch.bfloat16).to(DEV)
    s1, d1 = CreateSerde("cachegen", cfg, LMCacheEngineMetadata(name, 1, 0, "vllm"))
    s2, d2 = CreateSerde("cachegen", cfg, LMCacheEngineMetadata(name, 1, 0, "huggingface"))
    b1 = s1.to_bytes(kv)
    b2 = s2.to_bytes(kv.permute(0, 1, 3, 2, 4))
    assert len(b1) == len(b2)
    o = CacheGenEncoderOutput.from_bytes(b1)
    assert o.num_heads == 8 and o.head_size == 128 and len(o.data_chunks) == 1
    assert tuple(o.cdf.shape) == (64, 1024, 33) and tuple(o.max_tensors_key.shape) == (32, ntok, 1)
    r1 = d1.from_bytes(b1)
    r2 = d2.from_bytes(b2)
    assert r1.shape == kv.shape and r1.dtype == torch.bfloat16 and float(r1.float().mean()) != 0
    assert tuple(r2.shape) == (32, 2, 8, ntok, 128) and r2.dtype == torch.float16
    kb = s1.s.key_bins.cpu().numpy()
    vb = s1.s.value_bins.cpu().numpy()
    want = oracle.encode_function(bits(kv).reshape(32, 2, ntok, 1024), kb, vb, 1)
    _, want_kv = oracle.decode_function(want, kb, vb, max_dt=1, out_dt=1)
    assert np.array_equal(bits(r1).reshape(32, 2, ntok, 1024), want_kv)


# --------------------------------------------------------------------------- #
# wider tables and other bins tables (benchmark config 5 levels, 70B table)
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("kbins,vbins", [
    ([8.0] * 4, [8.0] * 4),                                   # level A: 8 bins everywhere
    ([16.0, 16.0, 16.0, 12.0], [16.0, 12.0, 12.0, 12.0]),      # level B: reference QUANT_LEVEL 1 tiers
    ([64.0, 32.0, 32.0, 32.0], [64.0, 32.0, 32.0, 32.0]),      # level D: 65-entry tables
    ([12.0, 10.0, 6.0, 4.0], [4.0, 6.0, 12.0, 12.0]),          # table lengths that are no power of two + 1
])
@pytest.mark.parametrize("rho", [0.5, 0.95])
def test_fused_path_other_bins_tables_match_oracle(oracle, kbins, vbins, rho):
    codec, _ = gpu_mods()
    from cachegen_amd.kvgen import make_kv
    L, T, H, D, S = 4, 600, 4, 64, 256
    kv = make_kv(L, T, H, D, seed=51, rho=rho)
    kb, vb = torch.tensor(kbins), torch.tensor(vbins)
    enc = codec.encode_kv(kv.to(DEV), kb.to(DEV), vb.to(DEV), chunk_tokens=S)
    enc.check()
    flat = bits(kv).reshape(L, 2, T, H * D)
    bounds = enc.sub_boundaries()
    out = codec.decode_encoded(enc, kb.to(DEV), vb.to(DEV), fmt="vllm", out_dtype=torch.float16)
    got = bits(out).reshape(L, 2, T, H * D)
    for i, t0 in enumerate(range(0, T, S)):
        t1 = min(t0 + S, T)
        want = oracle.encode_function(flat[:, :, t0:t1], kb.numpy(), vb.numpy())
        cdf, _, _, subs = enc.chunk(i, bounds)
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert np.array_equal(l.cpu().numpy(), wl) and np.array_equal(b.cpu().numpy(), wb)
        _, want_kv = oracle.decode_function(want, kb.numpy(), vb.numpy())
        assert np.array_equal(got[:, :, t0:t1], want_kv)
