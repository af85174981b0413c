"""An independent, bit-serial arithmetic coder on Python integers.

It is a second restatement of the algorithm, written from the older
one-bit-at-a-time form that the reference keeps beside the live kernels
(LMCache/third_party/torchac_cuda/torchac_kernel_enc.cu:15-45,194-375 for the
encoder and its bit sink; torchac_kernel_dec.cu:23-50,119-235 for the decoder
and its zero fill past the end of the stream).  The tests use it to check the
C oracle, whose encoder follows the 32-bit-register form of the live kernel;
the two share no code.
"""

M32 = 0xFFFFFFFF


class BitSink:
    def __init__(self):
        self.bits = []

    def bit_and_pending(self, bit, pending):
        self.bits.append(bit)
        self.bits.extend([1 - bit] * pending)

    def to_bytes(self):
        bits = list(self.bits)
        while len(bits) % 8:
            bits.append(0)
        out = bytearray()
        for i in range(0, len(bits), 8):
            b = 0
            for x in bits[i:i + 8]:
                b = (b << 1) | x
            out.append(b)
        return bytes(out)


def _bounds(cdf, s):
    lo = cdf[s]
    hi = 0x10000 if s == len(cdf) - 2 else cdf[s + 1]
    return lo, hi


def encode(cdf, symbols):
    """cdf: list of ints (length Lp); symbols: iterable of ints.  Returns (bytes, nbits)."""
    low, high, pending = 0, M32, 0
    sink = BitSink()
    for s in symbols:
        span = high - low + 1
        c_lo, c_hi = _bounds(cdf, s)
        high = (low - 1 + ((span * c_hi) >> 16)) & M32
        low = (low + ((span * c_lo) >> 16)) & M32
        while True:
            if high < 0x80000000:
                sink.bit_and_pending(0, pending)
                pending = 0
                low = (low << 1) & M32
                high = ((high << 1) & M32) | 1
            elif low >= 0x80000000:
                sink.bit_and_pending(1, pending)
                pending = 0
                low = (low << 1) & M32
                high = ((high << 1) & M32) | 1
            elif low >= 0x40000000 and high < 0xC0000000:
                pending += 1
                low = (low << 1) & 0x7FFFFFFF
                high = ((high << 1) & M32) | 0x80000001
            else:
                break
    pending += 1
    sink.bit_and_pending(0 if low < 0x40000000 else 1, pending)
    return sink.to_bytes(), len(sink.bits)


class BitSource:
    def __init__(self, data):
        self.data = data
        self.pos = 0

    def next(self):
        byte, off = divmod(self.pos, 8)
        self.pos += 1
        if byte >= len(self.data):
            return 0
        return (self.data[byte] >> (7 - off)) & 1


def _search(cdf, target):
    left, right = 0, len(cdf) - 1
    while left + 1 < right:
        m = (left + right) // 2
        if cdf[m] < target:
            left = m
        elif cdf[m] > target:
            right = m
        else:
            return m
    return left


def decode(cdf, data, n):
    src = BitSource(data)
    low, high, value = 0, M32, 0
    for _ in range(32):
        value = (value << 1) | src.next()
    out = []
    for i in range(n):
        span = high - low + 1
        count = (((value - low + 1) << 16) - 1) // span
        s = _search(cdf, count & 0xFFFF)
        out.append(s)
        if i == n - 1:
            break
        c_lo, c_hi = _bounds(cdf, s)
        high = (low - 1 + ((span * c_hi) >> 16)) & M32
        low = (low + ((span * c_lo) >> 16)) & M32
        while True:
            if low >= 0x80000000 or high < 0x80000000:
                low = (low << 1) & M32
                high = ((high << 1) & M32) | 1
                value = ((value << 1) & M32) | src.next()
            elif low >= 0x40000000 and high < 0xC0000000:
                low = (low << 1) & 0x7FFFFFFF
                high = ((high << 1) & M32) | 0x80000001
                value = (value - 0x40000000) & M32
                value = ((value << 1) & M32) | src.next()
            else:
                break
    return out
