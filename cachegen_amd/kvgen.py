"""Seeded synthetic KV caches with the statistics the benchmark configs name.

Per K/V layer each channel has a standard deviation drawn from LogNormal(0, 0.5);
2 % of the channels (chosen at random) are outliers with 10x that deviation; along
the token axis every channel is an AR(1) process with correlation `rho`:

    x_0 = sigma_c * e_0,   x_t = rho * x_{t-1} + sqrt(1 - rho^2) * sigma_c * e_t

The result is cast to 16 bits and laid out [L, 2, T, H, D] ("vllm" layout of
LMCache/lmcache/storage_backend/serde/cachegen_encoder.py:341-346).
"""
import torch


def make_kv(num_layers, num_tokens, num_heads, head_size, seed=1234, rho=0.9,
            device="cpu", dtype=torch.float16, outlier_frac=0.02, outlier_scale=10.0):
    """`rho` is a float, or a sequence of `num_layers` floats (one per layer)."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(int(seed))
    nc = num_heads * head_size
    rows = num_layers * 2
    sigma = torch.exp(0.5 * torch.randn(rows, nc, generator=gen, device=dev))
    n_out = max(1, int(round(outlier_frac * nc))) if outlier_frac > 0 else 0
    if n_out:
        pick = torch.rand(rows, nc, generator=gen, device=dev).argsort(dim=1)[:, :n_out]
        scale = torch.ones(rows, nc, device=dev)
        scale.scatter_(1, pick, outlier_scale)
        sigma = sigma * scale
    if isinstance(rho, (int, float)):
        rho_t = torch.full((rows, 1), float(rho), device=dev)
    else:
        assert len(rho) == num_layers
        rho_t = torch.tensor([float(r) for r in rho], device=dev).repeat_interleave(2)[:, None]
    innov = torch.sqrt(1.0 - rho_t * rho_t) * sigma
    out = torch.empty(num_layers, 2, num_tokens, nc, dtype=dtype, device=dev)
    flat = out.view(rows, num_tokens, nc)
    x = sigma * torch.randn(rows, nc, generator=gen, device=dev)
    flat[:, 0, :] = x.to(dtype)
    for t in range(1, num_tokens):
        x = rho_t * x + innov * torch.randn(rows, nc, generator=gen, device=dev)
        flat[:, t, :] = x.to(dtype)
    return out.view(num_layers, 2, num_tokens, num_heads, head_size)


def kv_nbytes(num_layers, num_tokens, num_heads, head_size):
    return 2 * num_layers * num_tokens * num_heads * head_size * 2


def entropy_bits(symbols, nbins):
    """Empirical zeroth-order entropy (bits per symbol) of an integer tensor."""
    counts = torch.bincount(symbols.flatten().to(torch.int64), minlength=nbins).double()
    p = counts[counts > 0] / counts.sum()
    return float(-(p * torch.log2(p)).sum())


__all__ = ["make_kv", "kv_nbytes", "entropy_bits"]
