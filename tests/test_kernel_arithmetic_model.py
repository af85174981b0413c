"""The HIP kernels do not run the reference's one-bit-at-a-time loops: they renormalise by a
shift count taken from two count-leading-zero operations, write the encoder's output as the
interval's lower end with carries instead of counting pending bits, track the decoder's code
value relative to the interval's low end, take the interval bounds from a high multiply and
leave bit 31 of `low` as it falls.  This module restates exactly
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


def bound_less_one(cdf, s, span_less_one):
    """The same from the encoder's state, which keeps span - 1 (2^32 - 1: full range): T(c) is the
    high word of span_less_one * (c << 16) + (c << 16), one 64-bit multiply-add (v_mad_u64_u32)
    with no case set apart for the full range."""
    def t(c):
        if c == 0x10000:
            return (span_less_one + 1) & M32               # 0 modulo 2^32 when the range is full
        total = span_less_one * (c << 16) + (c << 16)
        assert total < 1 << 64
        return total >> 32
    c_lo = cdf[s]
    c_hi = 0x10000 if s == len(cdf) - 2 else cdf[s + 1]
    return t(c_lo), (t(c_hi) - t(c_lo)) & M32


def shift_count(low, high):
    n1 = clz32(low ^ high)
    z = (((low & high) | (~low & M32)) << ((n1 + 1) & 31)) & M32
    return n1, clz32(z)


def model_encode(cdf, symbols, group=8):
    """RangeEncoder: the interval's lower end is one long number, `low` (its last 32 bits, the
    coder's window) below `out` (bits waiting to be written, at most 63 and a carry above them);
    a symbol adds its offset and shifts the number left by the step count; complete words leave
    once per `group` symbols through a held-back word that takes the carry, words of all ones
    being counted until the word after them shows whether a carry comes."""
    out, low, span_less_one, nout = 0, 0, M32, 0
    cache, ones, words, started = 0, 0, [], [False]

    def store(word):
        if not started[0]:                                 # the empty held-back word of the start
            started[0] = True
            assert word == 0
            return
        assert 0 <= word <= M32
        words.append(word)

    def release(carry):
        nonlocal ones
        store(cache + carry)
        for _ in range(ones):
            store(0 if carry else M32)
        ones = 0

    def flush_word():
        nonlocal out, nout, cache, ones
        sh = nout - 32
        word, carry = (out >> sh) & M32, out >> (sh + 32)
        assert carry in (0, 1)
        out &= (1 << sh) - 1
        nout = sh
        if ones == 0 and word != M32:
            store(cache + carry)
            cache = word
        elif carry:
            release(1)
            cache = word
        elif word == M32:
            ones += 1
        else:
            release(0)
            cache = word

    def add_low(t):
        nonlocal out, low
        total = low + t
        low, out = total & M32, out + (total >> 32)

    def shift(n):
        nonlocal out, low, nout
        if nout + n + 1 > 64:
            flush_word()
        big = ((out << 32) | low) << n
        low, out, nout = big & M32, big >> 32, nout + n
        assert out < 1 << 64

    for i, s in enumerate(symbols):
        t_lo, width = bound_less_one(cdf, s, span_less_one)
        assert (t_lo, width) == bound(cdf, s, (span_less_one + 1) & M32)
        add_low(t_lo)
        high = (low + width - 1) & M32                     # bit 31 of low may differ from the reference's
        n1, k = shift_count(low, high)
        shift(n1 + k)
        span_less_one = ((width << (n1 + k)) - 1) & M32
        if i % group == group - 1 and nout >= 32:
            flush_word()
    add_low(0x40000000)
    shift(2)
    if nout >= 32:
        flush_word()
    release(out >> nout)
    part = ((out & ((1 << nout) - 1)) << (32 - nout)) if nout else 0
    return b"".join(w.to_bytes(4, "big") for w in words) + part.to_bytes(4, "big")[:(nout + 7) // 8]


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


def test_carries_through_words_of_all_ones():
    """Streams whose lower end runs 0111...1 over several words (the reference counts hundreds of
    pending bits) and is then pushed over the edge, or not, by the symbols that follow."""
    for width in (1, 2, 5):
        cdf = [0, 65535 - width, 65535]
        for n in (3, 10, 40):
            for tail in ([], [0], [1, 0], [0, 0, 1]):
                syms = [1] * n + tail
                assert model_encode(cdf, syms) == pycoder.encode(cdf, syms)[0]
    cdf = [0, 32767, 32768, 65535]
    for n in range(1, 40):
        for last in (0, 1, 2):
            syms = [0] + [1] * n + [last, 2, 0, 1]
            want = pycoder.encode(cdf, syms)[0]
            assert model_encode(cdf, syms) == want
            assert model_decode(cdf, want, len(syms)) == syms


@pytest.mark.parametrize("group", [1, 2, 8])
def test_word_schedule_does_not_change_the_stream(group):
    rng = random.Random(group)
    for _ in range(30):
        nsym = rng.choice([3, 15, 31])
        cdf = random_table(rng, nsym, rng.choice([1, 8]))
        syms = [rng.randrange(nsym) for _ in range(rng.choice([5, 64, 300]))]
        assert model_encode(cdf, syms, group) == pycoder.encode(cdf, syms)[0]
