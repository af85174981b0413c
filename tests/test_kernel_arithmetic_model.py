"""The HIP kernels do not run the reference's one-bit-at-a-time loops: they renormalise by a
shift count taken from two count-leading-zero operations, splice pending bits in arithmetically,
track the decoder's code value relative to the interval's low end, take the interval bounds from
a high multiply and leave one bit of the decoder's `low` unmasked.  This module restates exactly
that arithmetic on Python integers (cachegen_amd/csrc/encoder.hpp: RangeEncoder::put_symbol,
decoder.hpp: decode_symbol) and checks it, on the CPU, against the independent bit-serial coder
of tests/pycoder.py: same bytes out of the encoder, same symbols out of the decoder, for tables
that provoke long underflow runs, full-range intervals and the last symbol's special bound."""
import random

import pytest

import pycoder

M32 = 0xFFFFFFFF


def clz32(x):
    return 32 - x.bit_length()


def bound(cdf, s, span):
    """T(c) for the lower and upper entry of symbol s; span is held modulo 2^32 (0: full range)."""
    def t(c):
        if c == 0x10000:
            return span                                    # 0 modulo 2^32 when the range is full
        if span == 0:
            return (c << 16) & M32
        return ((span * (c << 16)) >> 32) & M32            # v_mul_hi_u32(span, c << 16)
    c_lo = cdf[s]
    c_hi = 0x10000 if s == len(cdf) - 2 else cdf[s + 1]
    return t(c_lo), (t(c_hi) - t(c_lo)) & M32


def shift_count(low, high):
    n1 = clz32(low ^ high)
    z = (((low & high) | (~low & M32)) << ((n1 + 1) & 31)) & M32
    return n1, clz32(z)


def model_encode(cdf, symbols):
    bits = []                                              # emitted bits, as (value, count) pairs
    low, span, pend = 0, 0, 0
    for s in symbols:
        t_lo, width = bound(cdf, s, span)
        low = (low + t_lo) & M32
        high = (low + width - 1) & M32
        n1, k = shift_count(low, high)
        pe = pend if n1 > 0 else 0
        m = n1 + pe
        if n1 > 0:
            top = low >> (32 - n1)                         # v_bfe_u32(low, 32 - n1, n1)
            fill = ((1 << pe) - 1) << (n1 - 1)             # v_bfm_b32(pe, n1 - 1) when pe <= 31
            bits.append((top + fill, m))
        pend = pend - pe + k
        low = (low << (n1 + k)) & 0x7FFFFFFF
        span = (width << (n1 + k)) & M32
    pend += 1
    first = 0 if low < 0x40000000 else 1
    bits.append((first, 1))
    bits.append((0 if first else (1 << pend) - 1, pend))
    acc, nacc = 0, 0
    for v, m in bits:
        acc, nacc = (acc << m) | v, nacc + m
    pad = -nacc % 8
    return (acc << pad).to_bytes((nacc + pad) // 8, "big")


def model_decode(cdf, data, n):
    stream = int.from_bytes(data + b"\0" * 8, "big")
    total = 8 * (len(data) + 8)
    pos = 32

    def take(count):
        nonlocal pos
        v = (stream >> (total - pos - count)) & ((1 << count) - 1) if pos + count <= total else 0
        pos += count
        return v
    off = (stream >> (total - 32)) & M32
    low, span = 0, 0
    out = []
    for i in range(n):
        s = 0                                              # largest s with T(cdf[s]) <= off
        while s + 1 <= len(cdf) - 2 and bound(cdf, s + 1, span)[0] <= off:
            s += 1
        out.append(s)
        if i == n - 1:
            break
        t_lo, width = bound(cdf, s, span)
        assert (off - t_lo) & M32 < width or width == 0 and span == 0 and t_lo <= off
        low = (low + t_lo) & M32                           # bit 31 may hold a stale 1: never masked
        off -= t_lo
        high = (low + width - 1) & M32
        n1, k = shift_count(low, high)
        nshift = n1 + k
        low = (low << nshift) & M32
        span = (width << nshift) & M32
        off = ((off << nshift) | take(nshift)) & M32
    return out


def random_table(rng, nsym, skew):
    """Strictly increasing, first entry 0, top entry 65535 like calculate_cdf's; `skew` puts
    most of the mass on one symbol, which is what makes underflow runs long."""
    weights = [rng.random() ** skew + 1e-9 for _ in range(nsym)]
    weights[rng.randrange(nsym)] += skew * 20
    tot = sum(weights)
    cdf, run = [0], 0.0
    for i, w in enumerate(weights):
        run += w
        cdf.append(max(cdf[-1] + 1, min(65535 - (nsym - 1 - i), int(run / tot * (65535 - nsym)) + i + 1)))
    cdf[-1] = 65535
    return cdf


@pytest.mark.parametrize("seed", range(40))
def test_closed_form_coder_equals_bit_serial_coder(seed):
    rng = random.Random(seed)
    nsym = rng.choice([2, 3, 8, 15, 16, 31, 32, 63])
    cdf = random_table(rng, nsym, rng.choice([0.5, 1, 3, 8]))
    n = rng.choice([1, 2, 7, 64, 256])
    hot = max(range(nsym), key=lambda s: cdf[s + 1] - cdf[s])
    kind = rng.randrange(3)
    if kind == 0:
        syms = [rng.randrange(nsym) for _ in range(n)]
    elif kind == 1:                                        # mostly the likeliest symbol, rare others
        syms = [hot if rng.random() < 0.95 else rng.randrange(nsym) for _ in range(n)]
    else:                                                  # the last symbol (special upper bound) often
        syms = [nsym - 1 if rng.random() < 0.5 else rng.randrange(nsym) for _ in range(n)]
    want, _ = pycoder.encode(cdf, syms)
    assert model_encode(cdf, syms) == want
    assert model_decode(cdf, want, n) == syms
    assert pycoder.decode(cdf, want, n) == syms


def test_dyadic_table_hits_the_full_range_again():
    """Two symbols of probability 1/2 (cdf 0, 32768, 65536 = stored 65535 + special bound is not
    dyadic, so the half is built from entries 0 and 32768 of a three-symbol table): after a
    symbol of width exactly 2^31 the span renormalises to 2^32, i.e. 0 modulo 2^32."""
    cdf = [0, 32768, 65534, 65535]
    syms = [0, 0, 1, 0, 2, 0, 0, 1, 1, 0] * 5
    want, _ = pycoder.encode(cdf, syms)
    assert model_encode(cdf, syms) == want
    assert model_decode(cdf, want, len(syms)) == syms
