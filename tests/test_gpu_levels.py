"""Several quantization levels from one read of the tensor (cg_encode_kv_levels): every level's
tables, lengths, offsets and payload are byte-identical to a separate encode at that level, the
row maxima are shared, and one level goes through the oracle bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# the four levels of the adaptive-bitrate sweep, over (first, middle, last) tiers of 6 layers
LEVELS = [
    ([8.0] * 6, [8.0] * 6),
    ([16.0, 16.0, 16.0, 16.0, 12.0, 12.0], [16.0, 12.0, 12.0, 12.0, 12.0, 12.0]),
    ([32.0, 32.0, 16.0, 16.0, 16.0, 16.0], [32.0, 16.0, 16.0, 16.0, 16.0, 16.0]),
    ([64.0, 64.0, 32.0, 32.0, 32.0, 32.0], [64.0, 32.0, 32.0, 32.0, 32.0, 32.0]),
]


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _same(a, b):
    n = a.total_bytes()
    assert b.total_bytes() == n
    assert torch.equal(a.cdf, b.cdf) and torch.equal(a.lengths, b.lengths) and torch.equal(a.offsets, b.offsets)
    assert torch.equal(a.payload[:n], b.payload[:n]) and torch.equal(a.maxima, b.maxima)
    assert int(a.status) == int(b.status) == 0


@pytest.mark.parametrize("fmt", ["vllm", "huggingface"])
@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("shape,chunk", [((6, 700, 8, 128), 256), ((6, 700, 4, 64), 300), ((6, 130, 32, 128), 256),
                                         ((6, 90, 3, 20), 64)])
def test_levels_equal_separate_encodes(oracle, fmt, dtype, dt, shape, chunk):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    L, T, H, D = shape
    rho = [0.5 if l % 2 == 0 else 0.95 for l in range(L)]
    kv = make_kv(L, T, H, D, seed=77 + T, rho=rho, dtype=dtype)
    src = kv.to(DEV)
    if fmt == "huggingface":
        src = src.permute(0, 1, 3, 2, 4).contiguous()
    levels = [(torch.tensor(k), torch.tensor(v)) for k, v in LEVELS]
    print(dict(shape=shape, chunk=chunk, fmt=fmt, dtype=str(dtype)), flush=True)
    got = codec.encode_kv_levels(src, levels, chunk_tokens=chunk, fmt=fmt)
    assert len(got) == 4 and all(e.maxima.data_ptr() == got[0].maxima.data_ptr() for e in got)
    for (kb, vb), e in zip(levels, got):
        e.check()
        _same(e, codec.encode_kv(src, kb, vb, chunk_tokens=chunk, fmt=fmt))
    # one level against the oracle, chunk by chunk, and decoded
    v = 2
    kb, vb = LEVELS[v]
    kbn, vbn = np.array(kb, dtype=np.float32), np.array(vb, dtype=np.float32)
    flat = bits(kv).reshape(L, 2, T, H * D)
    bounds = got[v].sub_boundaries()
    out = codec.decode_encoded(got[v], levels[v][0], levels[v][1], fmt=fmt, out_dtype=dtype)
    dec = bits(out if fmt == "vllm" else out.permute(0, 1, 3, 2, 4)).reshape(L, 2, T, H * D)
    for i, t0 in enumerate(range(0, T, chunk)):
        t1 = min(t0 + chunk, T)
        want = oracle.encode_function(flat[:, :, t0:t1], kbn, vbn, dt)
        cdf, mk, mv, subs = got[v].chunk(i, bounds)
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"])
        assert np.array_equal(bits(mk)[..., 0], want["max_tensors_key"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert n == wn and np.array_equal(l.cpu().numpy(), wl) and np.array_equal(b.cpu().numpy(), wb)
        _, want_kv = oracle.decode_function(want, kbn, vbn, max_dt=dt, out_dt=dt)
        assert np.array_equal(dec[:, :, t0:t1], want_kv)
    # a second call into the same result and workspace gives the same bytes
    ws = torch.empty(codec.encode_levels_workspace_bytes(L, T, H * D, chunk, 4), dtype=torch.uint8, device=DEV)
    keep = [(e.cdf.clone(), e.lengths.clone(), e.payload[:e.total_bytes()].clone()) for e in got]
    again = codec.encode_kv_levels(src, levels, chunk_tokens=chunk, fmt=fmt, workspace=ws, out=got)
    assert again is got
    for e, (c, l, p) in zip(got, keep):
        assert torch.equal(e.cdf, c) and torch.equal(e.lengths, l) and torch.equal(e.payload[:p.numel()], p)


def test_levels_argument_checks():
    from cachegen_amd import codec
    kv = torch.zeros((2, 2, 16, 1, 8), dtype=torch.float16, device=DEV)
    b = torch.tensor([16.0, 16.0])
    with pytest.raises(RuntimeError, match="between 1 and 8 levels"):
        codec.encode_kv_levels(kv, [])
    with pytest.raises(RuntimeError, match="between 1 and 8 levels"):
        codec.encode_kv_levels(kv, [(b, b)] * 9)
    with pytest.raises(RuntimeError, match="one entry per layer"):
        codec.encode_kv_levels(kv, [(b, b[:1])])
    one = codec.encode_kv_levels(kv, [(b, b)])
    assert len(one) == 1 and int(one[0].status) == 0
