"""Delta-against-anchor token groups: an extension with NO counterpart in the reference
snapshot (it holds no anchor/delta code), so there is nothing to be bit-exact with.  The
definition lives in oracle/cachegen_oracle.c (cgo_quantize_delta / cgo_dequantize_delta);
it is pinned by a hand known-answer, by "groups of one are the plain codec" and by the
reconstruction bound; the HIP path is then compared with it bit for bit."""
import numpy as np
import pytest
import torch

DEV = "cuda:0"


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def test_delta_known_answer(oracle):
    # bins 32 -> MAX 15.  Row 0 is the anchor; row 1 is coded as d = row1 - row0 =
    # [0.25, 0, -0.25, 0.5]: max 0.5, factor 30, d*30+15 = [22.5, 15, 7.5, 30] -> [22, 15, 8, 30]
    x = np.array([[[1.0, -1.0, 0.5, 0.0], [1.25, -1.0, 0.25, 0.5]]], dtype=np.float16)
    sym, mx = oracle.quantize_delta(x.view(np.uint16), [32.0], group=10)
    assert sym[0].tolist() == [[30, 0, 22, 15], [22, 15, 8, 30]]
    assert mx.view(np.float16)[0].tolist() == [1.0, 0.5]
    out = oracle.dequantize_delta(sym, [32.0], mx, group=10).view(np.float16)
    f = np.float32
    anchor = np.array([1.0, -1.0, f(7) / f(15), 0.0], dtype=np.float32)
    delta = np.array([f(7) / f(15) * f(0.5), 0.0, f(-7) / f(15) * f(0.5), 0.5], dtype=np.float32)
    assert np.array_equal(out[0, 0], anchor.astype(np.float16))
    assert np.array_equal(out[0, 1], (delta + anchor).astype(np.float16))


def test_groups_of_one_are_the_plain_codec(oracle):
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(2, 300, 2, 16, seed=3)
    b = bits(kv).reshape(2, 2, 300, 32)
    bins = np.array([32.0, 16.0], dtype=np.float32)
    a = oracle.encode_function(b, bins, bins)
    d = oracle.encode_function(b, bins, bins, delta_group=1)
    assert np.array_equal(a["symbols"], d["symbols"]) and np.array_equal(a["cdf"], d["cdf"])
    assert np.array_equal(a["max_tensors_key"], d["max_tensors_key"])
    assert all(np.array_equal(x[0], y[0]) for x, y in zip(a["data_chunks"], d["data_chunks"]))
    _, ka = oracle.decode_function(a, bins, bins)
    _, kd = oracle.decode_function(d, bins, bins, delta_group=1)
    assert np.array_equal(ka, kd)


def test_delta_reconstruction_bound(oracle):
    """|x^ - x| <= step_anchor/2 + step_delta/2 per element (plus 16-bit rounding).  Every row is
    scaled by its own maximum and every delta row inherits its anchor's error, so on the
    benchmark's generator the mode changes neither size nor error by much; only the bound and
    a sane size are asserted."""
    from cachegen_amd.kvgen import make_kv
    L, T, C = 2, 512, 64
    kv = make_kv(L, T, 2, 32, seed=8, rho=0.98, outlier_frac=0.0)
    b = bits(kv).reshape(L, 2, T, C)
    bins = np.array([32.0, 32.0], dtype=np.float32)
    plain = oracle.encode_function(b, bins, bins)
    delta = oracle.encode_function(b, bins, bins, delta_group=10)
    _, out = oracle.decode_function(delta, bins, bins, delta_group=10)
    x = kv.reshape(L, 2, T, C).float().numpy()
    y = out.view(np.float16).astype(np.float32)
    mk = np.stack([delta["max_tensors_key"], delta["max_tensors_value"]], axis=1).view(np.float16).astype(np.float32)
    step = mk / 15.0                                      # [L, 2, T]
    t = np.arange(T)
    anchor_t = t - (t % 256) % 10
    bound = 0.5 * step + np.where(anchor_t == t, 0.0, 0.5 * step[:, :, anchor_t])
    assert (np.abs(x - y) <= bound[..., None] * 1.02 + 2e-3 * np.abs(x)).all()
    size = lambda e: sum(len(c[0]) for c in e["data_chunks"])
    assert size(delta) < 1.25 * size(plain)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,dt", [(torch.float16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("L,T,H,D,S,G", [(2, 512, 8, 64, 512, 10), (2, 300, 4, 32, 300, 10),
                                         (3, 700, 2, 64, 256, 7), (1, 520, 16, 128, 260, 256)])
def test_hip_delta_groups_match_oracle(oracle, dtype, dt, L, T, H, D, S, G):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(L, T, H, D, seed=61 + T, dtype=dtype)
    kv[0, 0, 5] = 0
    kb = torch.tensor([32.0, 16.0, 12.0][:L])
    vb = torch.tensor([32.0, 32.0, 16.0][:L]) if L > 1 else torch.tensor([32.0])
    if L == 1:
        kb = torch.tensor([32.0])
    enc = codec.encode_kv(kv.to(DEV), kb.to(DEV), vb.to(DEV), chunk_tokens=S, delta_group=G)
    enc.check()
    flat = bits(kv).reshape(L, 2, T, H * D)
    bounds = enc.sub_boundaries()
    out = codec.decode_encoded(enc, kb.to(DEV), vb.to(DEV), fmt="vllm", out_dtype=dtype)
    got = bits(out).reshape(L, 2, T, H * D)
    for i, t0 in enumerate(range(0, T, S)):
        t1 = min(t0 + S, T)
        want = oracle.encode_function(flat[:, :, t0:t1], kb.numpy(), vb.numpy(), dt, delta_group=G)
        cdf, mk, mv, subs = enc.chunk(i, bounds)
        assert np.array_equal(bits(mk)[..., 0], want["max_tensors_key"])
        assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"])
        for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
            assert np.array_equal(l.cpu().numpy(), wl) and np.array_equal(b.cpu().numpy(), wb)
        _, want_kv = oracle.decode_function(want, kb.numpy(), vb.numpy(), max_dt=dt, out_dt=dt, delta_group=G)
        assert np.array_equal(got[:, :, t0:t1], want_kv)


@pytest.mark.gpu
def test_hip_delta_off_is_the_plain_path():
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    kv = make_kv(2, 512, 8, 64, seed=5).to(DEV)
    b = torch.tensor([32.0, 16.0], device=DEV)
    a = codec.encode_kv(kv, b, b, chunk_tokens=256)
    d = codec.encode_kv(kv, b, b, chunk_tokens=256, delta_group=1)
    n = a.total_bytes()
    assert d.total_bytes() == n and torch.equal(a.payload[:n], d.payload[:n]) and torch.equal(a.cdf, d.cdf)
    assert torch.equal(a.maxima, d.maxima)
