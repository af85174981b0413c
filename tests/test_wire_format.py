"""The flat wire container (cachegen_amd/serde/wire.py): layout known answers and validation
on the CPU, and on the GPU the equality of the device-assembled blobs with the host
definition and of the decoded tensors with the pickle container's."""
import pickle
import struct

import numpy as np
import pytest
import torch

from cachegen_amd.serde import wire


def _small_arrays(rng, L=1, T=300, H=1, D=2, S=300, lp=5):
    C = H * D
    nchunks = -(-T // S)
    nsub = wire.geometry(L, T, H, D, S, lp - 1, 0)["nsub"][0]
    cdf = rng.integers(0, 65536, size=(nchunks, 2 * L, C, lp), dtype=np.uint16)
    maxima = rng.integers(0, 65536, size=(2, L, T), dtype=np.uint16)
    lengths = rng.integers(1, 200, size=(nsub, 2 * L, C)).astype(np.int32)
    payload = rng.integers(0, 256, size=int(lengths.sum()), dtype=np.uint8)
    return cdf, maxima, lengths, payload


def test_layout_known_answer():
    """L=1, T=300, H=1, D=2, one table: sections at 64, 64+40->128, 128+1200->1344, 1344+32->1408."""
    rng = np.random.default_rng(0)
    cdf, maxima, lengths, payload = _small_arrays(rng)
    assert cdf.nbytes == 40 and maxima.nbytes == 1200 and lengths.nbytes == 32
    blob = wire.pack_host(cdf, maxima, lengths, payload, num_heads=1, head_size=2, chunk_tokens=300)
    assert blob[:4] == b"CGKV"
    assert struct.unpack_from("<HH", blob, 4) == (1, 0)
    assert struct.unpack_from("<8I", blob, 8) == (1, 300, 1, 2, 300, 4, 0, 2)
    assert struct.unpack_from("<Q", blob, 40) == (payload.size,)
    assert blob[48:64] == bytes(16)
    assert blob[64:104] == cdf.tobytes() and blob[104:128] == bytes(24)
    assert blob[128:1328] == maxima.tobytes() and blob[1328:1344] == bytes(16)
    assert blob[1344:1376] == lengths.tobytes()
    assert blob[1408:1408 + payload.size] == payload.tobytes()
    assert len(blob) == 1408 + (payload.size + 63) // 64 * 64
    assert wire.is_flat(blob) and not wire.is_flat(pickle.dumps({"a": 1})) and not wire.is_flat(b"")


@pytest.mark.parametrize("T,S", [(300, 300), (700, 256), (1500, 1500), (1501, 600)])
def test_host_round_trip(T, S):
    rng = np.random.default_rng(T)
    cdf, maxima, lengths, payload = _small_arrays(rng, L=2, T=T, H=2, D=3, S=S, lp=17)
    blob = wire.pack_host(cdf, maxima, lengths, payload, 2, 3, S, delta_group=4, bf16_maxima=True)
    h, c2, m2, l2, p2 = wire.unpack_host(blob)
    assert (h["num_layers"], h["num_tokens"], h["num_heads"], h["head_size"]) == (2, T, 2, 3)
    assert (h["chunk_tokens"], h["max_bins"], h["delta_group"], h["bf16_maxima"]) == (S, 16, 4, True)
    for a, b in ((cdf, c2), (maxima, m2), (lengths, l2), (payload, p2)):
        assert a.dtype == b.dtype and np.array_equal(a, b)


def test_sub_chunk_count_follows_the_chunking():
    # 1501 tokens cut every 600: chunks of 600, 600, 301 tokens -> 3 + 3 + 2 sub-chunks
    assert wire.geometry(1, 1501, 1, 1, 600, 4, 0)["nsub"][0] == 8
    assert wire.geometry(1, 1501, 1, 1, 600, 4, 0)["nchunks"][0] == 3
    assert wire.geometry(1, 256, 1, 1, 256, 4, 0)["nsub"][0] == 1


def test_invalid_blobs_are_rejected():
    rng = np.random.default_rng(3)
    cdf, maxima, lengths, payload = _small_arrays(rng)
    blob = wire.pack_host(cdf, maxima, lengths, payload, 1, 2, 300)
    with pytest.raises(ValueError, match="bad magic"):
        wire.read_header(b"XXXX" + blob[4:])
    with pytest.raises(ValueError, match="version"):
        wire.read_header(blob[:4] + struct.pack("<H", 9) + blob[6:])
    with pytest.raises(ValueError, match="unknown flags"):
        wire.read_header(blob[:6] + struct.pack("<H", 0x80) + blob[8:])
    with pytest.raises(ValueError, match="geometry gives"):
        wire.read_header(blob[:-64])
    with pytest.raises(ValueError, match="shorter than its header"):
        wire.read_header(blob[:10])
    with pytest.raises(ValueError, match="sub-chunks recorded"):
        wire.read_header(blob[:36] + struct.pack("<I", 3) + blob[40:])
    bad = bytearray(blob)
    bad[1344:1348] = struct.pack("<i", int(lengths.flat[0]) + 1)      # one length no longer matches
    with pytest.raises(ValueError, match="sum of the stream lengths"):
        wire.unpack_host(bytes(bad))
    with pytest.raises(ValueError, match="sum of the stream lengths"):
        wire.pack_host(cdf, maxima, lengths, payload[:-1], 1, 2, 300)
    with pytest.raises(ValueError, match="shapes do not agree"):
        wire.pack_host(cdf, maxima, lengths, payload, 1, 3, 300)


# --------------------------------------------------------------------------- #
# GPU
# --------------------------------------------------------------------------- #
DEV = "cuda:0"


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_device_blobs_equal_the_host_definition(dtype):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    L, T, H, D, S = 2, 900, 4, 64, 512
    kv = make_kv(L, T, H, D, seed=11, device=DEV, dtype=dtype)
    bins = torch.tensor([32.0, 16.0])
    enc = codec.encode_kv(kv, bins, bins, chunk_tokens=S)
    blobs = wire.pack_chunks(enc)
    assert len(blobs) == 2
    bounds = enc.sub_boundaries()
    for i, blob in enumerate(blobs):
        t0, t1 = i * S, min((i + 1) * S, T)
        g0, g1 = 2 * i, min(2 * i + 2, enc.lengths.shape[0])
        want = wire.pack_host(enc.cdf[i:i + 1].cpu().numpy(), _bits(enc.maxima[:, :, t0:t1]),
                              enc.lengths[g0:g1].cpu().numpy(), enc.payload[bounds[g0]:bounds[g1]].cpu().numpy(),
                              H, D, min(S, t1 - t0), bf16_maxima=dtype == torch.bfloat16)
        assert blob == want
    whole = wire.pack_chunks(enc, per_chunk=False)
    assert len(whole) == 1
    want = wire.pack_host(enc.cdf.cpu().numpy(), _bits(enc.maxima), enc.lengths.cpu().numpy(),
                          enc.payload[:enc.total_bytes()].cpu().numpy(), H, D, S,
                          bf16_maxima=dtype == torch.bfloat16)
    assert whole[0] == want
    # back on the device: the sections are the encoder's tensors
    h, cdf, maxima, lengths, payload = wire.unpack_to_device(whole[0], DEV)
    assert torch.equal(cdf, enc.cdf) and torch.equal(lengths, enc.lengths)
    assert maxima.dtype == dtype and torch.equal(maxima.view(torch.int16), enc.maxima.view(torch.int16))
    assert torch.equal(payload, enc.payload[:enc.total_bytes()])
    out = codec.decode_kv(cdf, maxima, codec.scan_lengths(lengths), payload, bins, bins, L, T, H, D, S,
                          out_dtype=dtype)
    assert torch.equal(out.view(torch.int16), codec.decode_encoded(enc, bins, bins, out_dtype=dtype).view(torch.int16))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
def test_flat_serde_decodes_to_the_same_tensor_as_the_pickle_serde(fmt):
    from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import CreateSerde
    config = LMCacheEngineConfig.from_defaults(chunk_size=256)
    meta = LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, 0, fmt)
    s_ref, d = CreateSerde("cachegen", config, meta)
    s_flat, _ = CreateSerde("cachegen-flat", config, meta)
    for ntok in (256, 77, 600):
        kv = make_kv(32, ntok, 2, 64, seed=ntok, device=DEV)
        if fmt == "huggingface":
            kv = kv.permute(0, 1, 3, 2, 4).contiguous()
        a, b = s_ref.to_bytes(kv), s_flat.to_bytes(kv)
        assert wire.is_flat(b) and not wire.is_flat(a)
        assert len(b) < len(a) + 512 and len(a) < len(b) + 8192     # neither container carries dead bytes
        ta, tb = d.from_bytes(a), d.from_bytes(b)
        assert ta.shape == kv.shape and ta.dtype == tb.dtype
        assert torch.equal(ta.view(torch.int16), tb.view(torch.int16))
    bad = bytearray(b)
    h = wire.read_header(b)
    off = h["geometry"]["lengths"][0]
    bad[off:off + 4] = struct.pack("<i", 1 + struct.unpack_from("<i", b, off)[0])
    with pytest.raises(ValueError, match="sum of the stream lengths"):
        d.from_bytes(bytes(bad))


# --------------------------------------------------------------------------- #
# version 2: tables as histogram counts
# --------------------------------------------------------------------------- #
def _histogram_case(rng, tokens, rows=4, C=5, nsyms=32):
    counts = np.zeros((len(tokens), rows, C, nsyms), dtype=np.int64)
    for c, n in enumerate(tokens):
        for r in range(rows):
            top = [15, 31, 7, 32][r % 4]
            for ch in range(C):
                syms = rng.integers(0, top, size=n)
                if r == 2 and ch == 0:
                    syms[:] = 3                                   # one symbol for the whole chunk
                counts[c, r, ch] = np.bincount(syms, minlength=nsyms)
    return counts


def test_tables_are_recovered_from_their_histograms():
    rng = np.random.default_rng(5)
    tokens = [256, 256, 77]
    counts = _histogram_case(rng, tokens)
    cdf = wire.counts_to_tables(counts, tokens)
    # known answer (the CDF example of 4 symbols [0, 0, 1, 30] over 32 levels)
    one = np.zeros((1, 1, 1, 32), dtype=np.int64)
    one[0, 0, 0, [0, 1, 30]] = [2, 1, 1]
    want = [0, 32752] + [49127 + i for i in range(2, 31)] + [65534, 65535]
    assert wire.counts_to_tables(one, [4])[0, 0, 0].tolist() == want
    assert np.array_equal(wire.tables_to_counts(cdf, tokens), counts)
    nsym, data = wire.pack_counts(counts)
    assert nsym.tolist() == [[15, 31, 7, 32]] * 3
    assert data.size == 3 * 5 * (15 + 31 + 7 + 32) and int(data.max()) == 255      # the 256 is clamped
    assert np.array_equal(wire.unpack_counts(nsym, data, 5, 32, tokens), counts)
    # a table that no histogram produces is refused
    bad = cdf.copy()
    bad[0, 0, 0, 5] += 1
    assert wire.tables_to_counts(bad, tokens) is None


@pytest.mark.parametrize("T,S", [(256, 256), (600, 256), (100, 100)])
def test_compact_host_round_trip(T, S):
    rng = np.random.default_rng(T)
    tokens = wire.chunk_token_counts(T, S)
    counts = _histogram_case(rng, tokens, rows=4, C=6, nsyms=32)
    cdf = wire.counts_to_tables(counts, tokens)
    nsub = wire.geometry(2, T, 2, 3, S, 32, 0)["nsub"][0]
    maxima = rng.integers(0, 65536, size=(2, 2, T), dtype=np.uint16)
    lengths = rng.integers(1, 200, size=(nsub, 4, 6)).astype(np.int32)
    payload = rng.integers(0, 256, size=int(lengths.sum()), dtype=np.uint8)
    flat = wire.pack_host(cdf, maxima, lengths, payload, 2, 3, S)
    compact = wire.pack_host(cdf, maxima, lengths, payload, 2, 3, S, compact=True)
    assert len(compact) < len(flat)
    h, c2, m2, l2, p2 = wire.unpack_host(compact)
    assert h["version"] == 2 and h["count_tables"] and h["lengths_u16"]
    for a, b in ((cdf, c2), (maxima, m2), (lengths, l2), (payload, p2)):
        assert np.array_equal(a, b)
    # corrupt one count: the chunk's tokens no longer add up
    off = h["geometry"]["cdf"][0] + len(tokens) * 4
    bad = bytearray(compact)
    bad[off] = (bad[off] + 1) % 200
    with pytest.raises(ValueError, match="add up"):
        wire.unpack_host(bytes(bad))


def test_compact_falls_back_to_raw_tables_and_wide_lengths():
    rng = np.random.default_rng(9)
    cdf, maxima, lengths, payload = _small_arrays(rng, L=1, T=200, H=1, D=2, S=200, lp=17)   # arbitrary tables
    blob = wire.pack_host(cdf, maxima, lengths, payload, 1, 2, 200, compact=True)
    h, c2, _, l2, _ = wire.unpack_host(blob)
    assert h["version"] == 2 and not h["count_tables"] and h["lengths_u16"]
    assert np.array_equal(c2, cdf) and np.array_equal(l2, lengths)
    # chunks longer than 256 tokens keep raw tables as well
    cdf, maxima, lengths, payload = _small_arrays(rng, L=1, T=700, H=1, D=2, S=700, lp=9)
    h, c2, _, _, _ = wire.unpack_host(wire.pack_host(cdf, maxima, lengths, payload, 1, 2, 700, compact=True))
    assert not h["count_tables"] and np.array_equal(c2, cdf)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_compact_device_blobs_equal_the_host_definition(dtype):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    L, T, H, D, S = 3, 600, 4, 64, 256
    kv = make_kv(L, T, H, D, seed=12, device=DEV, dtype=dtype)
    kv[1, 0, 256:512] = 0                                  # all-zero rows: one symbol for whole chunks
    kb, vb = torch.tensor([32.0, 16.0, 12.0]), torch.tensor([32.0, 8.0, 32.0])
    enc = codec.encode_kv(kv, kb, vb, chunk_tokens=S)
    bounds = enc.sub_boundaries()
    blobs = wire.pack_chunks(enc, compact=True)
    flat = wire.pack_chunks(enc)
    assert len(blobs) == 3
    for i, blob in enumerate(blobs):
        t0, t1 = i * S, min((i + 1) * S, T)
        want = wire.pack_host(enc.cdf[i:i + 1].cpu().numpy(), _bits(enc.maxima[:, :, t0:t1]),
                              enc.lengths[i:i + 1].cpu().numpy(), enc.payload[bounds[i]:bounds[i + 1]].cpu().numpy(),
                              H, D, min(S, t1 - t0), bf16_maxima=dtype == torch.bfloat16, compact=True)
        assert blob == want
        assert wire.read_header(blob)["count_tables"] and len(blob) < 0.75 * len(flat[i])
        h, cdf, maxima, lengths, payload = wire.unpack_to_device(blob, DEV)
        assert torch.equal(cdf, enc.cdf[i:i + 1]) and torch.equal(lengths, enc.lengths[i:i + 1])
        assert torch.equal(payload, enc.payload[bounds[i]:bounds[i + 1]])
    whole = wire.pack_chunks(enc, per_chunk=False, compact=True)[0]
    h, cdf, maxima, lengths, payload = wire.unpack_to_device(whole, DEV)
    assert torch.equal(cdf, enc.cdf) and torch.equal(lengths, enc.lengths)
    out = codec.decode_kv(cdf, maxima, codec.scan_lengths(lengths), payload, kb, vb, L, T, H, D, S, out_dtype=dtype)
    assert torch.equal(out.view(torch.int16), codec.decode_encoded(enc, kb, vb, out_dtype=dtype).view(torch.int16))


@pytest.mark.gpu
def test_compact_serde_decodes_like_the_pickle_serde():
    from cachegen_amd.config import LMCacheEngineConfig, LMCacheEngineMetadata
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import CreateSerde
    config = LMCacheEngineConfig.from_defaults(chunk_size=256)
    for fmt in ("vllm", "huggingface"):
        meta = LMCacheEngineMetadata("lmsys/longchat-7b-16k", 1, 0, fmt)
        s_ref, d = CreateSerde("cachegen", config, meta)
        s_small, _ = CreateSerde("cachegen-compact", config, meta)
        for ntok in (256, 31, 600):
            kv = make_kv(32, ntok, 2, 64, seed=ntok + 1, device=DEV)
            if fmt == "huggingface":
                kv = kv.permute(0, 1, 3, 2, 4).contiguous()
            a, b = s_ref.to_bytes(kv), s_small.to_bytes(kv)
            assert wire.read_header(b)["version"] == 2
            assert wire.read_header(b)["count_tables"] == (ntok <= 256)
            if ntok <= 256:
                assert len(b) < 0.75 * len(a)
            assert torch.equal(d.from_bytes(a), d.from_bytes(b))


@pytest.mark.gpu
def test_corrupt_compact_blob_is_rejected_on_the_device():
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(2, 256, 2, 64, seed=3, device=DEV)
    bins = torch.tensor([32.0, 16.0])
    enc = codec.encode_kv(kv, bins, bins, chunk_tokens=256)
    blob = wire.pack_chunks(enc, compact=True)[0]
    h = wire.read_header(blob)
    assert h["count_tables"]
    off = h["geometry"]["cdf"][0]
    bad = bytearray(blob)
    bad[off + 4 + 7] = (bad[off + 4 + 7] + 1) % 200        # one histogram count (4 bytes of nsym come first)
    with pytest.raises(ValueError, match="add up"):
        wire.unpack_to_device(bytes(bad), DEV)
    bad = bytearray(blob)
    bad[off] = 200                                         # a symbol count beyond the table
    with pytest.raises(ValueError, match="outside the table"):
        wire.unpack_to_device(bytes(bad), DEV)
    bad = bytearray(blob)
    bad[off] = max(1, bad[off] - 1)                        # a symbol count that no longer matches the section size
    with pytest.raises(ValueError, match="does not match"):
        wire.unpack_to_device(bytes(bad), DEV)
