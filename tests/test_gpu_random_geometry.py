"""Seeded sweep over random geometries, level tables, dtypes and layouts: the fused HIP path
against the oracle, bit for bit.  Shapes are drawn to hit the branches of the host code (packed
and byte symbols, fused and separate tables, partial channel tiles, ragged chunks, block sizes,
table lengths with and without an unrolled decoder, strided inputs and outputs)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
LEVELS = [8, 12, 16, 24, 32, 48, 64]


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def draw_case(rng, wide=False):
    L = int(rng.integers(1, 5))
    H = int(rng.choice([1, 2, 3, 4, 8]))
    D = int(rng.choice([8, 16, 20, 32, 40, 64, 128]))
    T = int(rng.integers(1, 900))
    if wide:
        # 1280 to 4096 channels: the fused quantiser's four and eight loads per lane, many
        # channel tiles per row, a partial last tile (1280 = 5 x 256, 3072 = 12 x 256 are whole;
        # 24 x 72 = 1728 is not)
        L = int(rng.integers(1, 4))
        H, D = [(16, 128), (32, 128), (32, 64), (24, 72), (10, 128), (24, 128)][int(rng.integers(0, 6))]
        T = int(rng.integers(1, 600))
    S = int(rng.choice([T, 256, int(rng.integers(1, T + 1)), 300, 512]))
    top = int(rng.choice(LEVELS))
    lower = [b for b in LEVELS if b <= top]
    kb = rng.choice(lower, size=L).astype(np.float32)
    vb = rng.choice(lower, size=L).astype(np.float32)
    kb[int(rng.integers(0, L))] = top                    # both tables reach the same maximum,
    vb[int(rng.integers(0, L))] = top                    # as the reference's torch.cat needs
    dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
    fmt = ["vllm", "huggingface"][int(rng.integers(0, 2))]
    kind = int(rng.integers(0, 3))                       # 0 generator, 1 white noise, 2 sparse with zeros
    return L, T, H, D, S, kb, vb, dtype, fmt, kind


@pytest.mark.parametrize("seed", range(12))
def test_random_case_matches_oracle(oracle, seed):
    run_cases(oracle, seed, 4, False)


@pytest.mark.parametrize("seed", range(100, 106))
def test_random_wide_case_matches_oracle(oracle, seed):
    run_cases(oracle, seed, 2, True)


@pytest.mark.parametrize("seed", range(12, 24))
def test_random_case_with_tables_built_by_the_quantizer(oracle, seed):
    """The same sweep with the form of cg_encode_kv that small calls do not take by themselves
    forced through the library's test entry point (CG_TEST_TABLES_IN_QUANTIZER); shapes the form
    does not cover (table lengths other than 9, 17, 33, 65; more than 2048 channels) fall back."""
    run_cases(oracle, seed, 4, False, flags=2)


@pytest.mark.parametrize("seed", range(106, 110))
def test_random_wide_case_with_tables_built_by_the_quantizer(oracle, seed):
    run_cases(oracle, seed, 2, True, flags=2)


@pytest.mark.parametrize("seed", range(24, 32))
def test_random_case_with_chunks_counted_in_parts(oracle, seed):
    """The quantizer-built tables with every chunk of more than 256 tokens cut into parts of 256
    tokens that separate blocks count (CG_TEST_SPLIT_CHUNKS), as calls with few long chunks do."""
    run_cases(oracle, seed, 4, False, flags=2 | 8)


def run_cases(oracle, seed, ncases, wide, flags=None):
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    rng = np.random.default_rng(9000 + seed)
    for _ in range(ncases):
        L, T, H, D, S, kb, vb, dtype, fmt, kind = draw_case(rng, wide)
        label = dict(L=L, T=T, H=H, D=D, S=S, kb=kb.tolist(), vb=vb.tolist(), dtype=str(dtype), fmt=fmt, kind=kind)
        print(label, flush=True)
        gen = torch.Generator().manual_seed(seed * 100 + T)
        if kind == 0:
            kv = make_kv(L, T, H, D, seed=seed * 7 + T, dtype=dtype)
        elif kind == 1:
            kv = torch.randn((L, 2, T, H, D), generator=gen).to(dtype)
        else:
            kv = torch.randn((L, 2, T, H, D), generator=gen)
            kv = (kv * (torch.rand((L, 2, T, H, D), generator=gen) < 0.2)).to(dtype)
            kv[:, :, T // 2] = 0                                           # one all-zero row per layer
        dt = 0 if dtype == torch.float16 else 1
        C = H * D
        flat = bits(kv).reshape(L, 2, T, C)
        # hand the kernels a strided view: the tensor sits inside a larger one
        dev_kv = kv.to(DEV)
        if fmt == "huggingface":
            big = torch.zeros((L, 2, H, T + 3, D), dtype=dtype, device=DEV)
            big[:, :, :, 2:2 + T] = dev_kv.permute(0, 1, 3, 2, 4)
            src = big[:, :, :, 2:2 + T]
        else:
            big = torch.zeros((L, 2, T + 3, H, D), dtype=dtype, device=DEV)
            big[:, :, 1:1 + T] = dev_kv
            src = big[:, :, 1:1 + T]
        kbt, vbt = torch.from_numpy(kb), torch.from_numpy(vb)
        enc = codec.encode_kv(src, kbt, vbt, chunk_tokens=S, fmt=fmt, _test_flags=flags)
        enc.check()
        bounds = enc.sub_boundaries()
        out_dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
        odt = 0 if out_dtype == torch.float16 else 1
        out = codec.decode_encoded(enc, kbt, vbt, fmt=fmt, out_dtype=out_dtype)
        got = out if fmt == "vllm" else out.permute(0, 1, 3, 2, 4)
        got = bits(got).reshape(L, 2, T, C)
        for i, t0 in enumerate(range(0, T, S)):
            t1 = min(t0 + S, T)
            want = oracle.encode_function(flat[:, :, t0:t1], kb, vb, dt)
            cdf, max_k, max_v, subs = enc.chunk(i, bounds)
            assert np.array_equal(cdf.cpu().numpy().view(np.uint16), want["cdf"]), label
            assert np.array_equal(bits(max_k)[..., 0], want["max_tensors_key"]), label
            assert np.array_equal(bits(max_v)[..., 0], want["max_tensors_value"]), label
            assert len(subs) == len(want["data_chunks"]), label
            for (b, l, n), (wb, wl, wn) in zip(subs, want["data_chunks"]):
                assert n == wn and np.array_equal(l.cpu().numpy(), wl), label
                assert np.array_equal(b.cpu().numpy(), wb), label
            _, want_kv = oracle.decode_function(want, kb, vb, max_dt=dt, out_dt=odt)
            assert np.array_equal(got[:, :, t0:t1], want_kv), label
