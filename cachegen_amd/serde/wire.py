"""Flat wire container for encoded KV chunks.

The reference ships a chunk as a pickle of `CacheGenGPUEncoderOutput` holding GPU tensors
(LMCache/lmcache/storage_backend/serde/cachegen_basics.py:110-122): one device-to-host copy
per tensor when it is written, code execution from the blob when it is read.  This container
carries the same fields in one flat, versioned, little-endian buffer, so that a chunk is one
device-to-host copy out of a staging buffer and one host-to-device copy back, and reading it
executes nothing.  `CacheGenDeserializer.from_bytes` accepts both forms (it looks at the
first four bytes); the pickle form stays the default for drop-in use.

Layout (every section starts on a 64-byte boundary; the gaps are zero):

    header   64 bytes   see HEADER
    cdf      int16  [nchunks, 2L, C, max_bins + 1]
    maxima   16-bit [2, L, T]           (float16 or bfloat16 bit patterns, see flags)
    lengths  int32  [nsub, 2L, C]       bytes of every stream, in stream order
    payload  uint8  [payload_bytes]     all streams back to back

Stream offsets are not stored: they are the running sum of `lengths`, which the decoder
recomputes on the GPU exactly as cachegen_decoder.py:70 does.  A stream longer than 256
bytes is stored cut to 256 (its length field keeps the full value), as in the device format.
"""
import struct
from typing import Dict, List, Optional, Tuple

import numpy as np

MAGIC = b"CGKV"
VERSION = 1
ALIGN = 64
HEADER_BYTES = 64
# magic, version, flags, L, T, H, D, chunk_tokens, max_bins, delta_group, nsub, payload_bytes
HEADER = struct.Struct("<4sHHIIIIIIIIQ")
FLAG_BF16_MAXIMA = 1
MAX_STREAM_BYTES = 256


def _up(n: int) -> int:
    return (n + ALIGN - 1) // ALIGN * ALIGN


def is_flat(blob) -> bool:
    return len(blob) >= 4 and bytes(blob[:4]) == MAGIC


def geometry(num_layers: int, num_tokens: int, num_heads: int, head_size: int, chunk_tokens: int,
             max_bins: int, payload_bytes: int) -> Dict[str, Tuple[int, int]]:
    """Section name -> (byte offset, byte size), plus "total" -> (size of the blob, 0)."""
    if min(num_layers, num_tokens, num_heads, head_size, chunk_tokens, max_bins) <= 0 or payload_bytes < 0:
        raise ValueError("wire container: sizes must be positive")
    C = num_heads * head_size
    nchunks = -(-num_tokens // chunk_tokens)
    full, rest = divmod(num_tokens, chunk_tokens)
    nsub = full * (-(-chunk_tokens // MAX_STREAM_BYTES)) + (-(-rest // MAX_STREAM_BYTES))
    sizes = [("cdf", nchunks * 2 * num_layers * C * (max_bins + 1) * 2),
             ("maxima", 2 * num_layers * num_tokens * 2),
             ("lengths", nsub * 2 * num_layers * C * 4),
             ("payload", payload_bytes)]
    out, pos = {}, HEADER_BYTES
    for name, size in sizes:
        out[name] = (pos, size)
        pos = _up(pos + size)
    out["total"] = (pos, 0)
    out["nsub"] = (nsub, 0)
    out["nchunks"] = (nchunks, 0)
    return out


def write_header(num_layers, num_tokens, num_heads, head_size, chunk_tokens, max_bins, delta_group,
                 nsub, payload_bytes, bf16_maxima) -> bytes:
    head = HEADER.pack(MAGIC, VERSION, FLAG_BF16_MAXIMA if bf16_maxima else 0, num_layers, num_tokens,
                       num_heads, head_size, chunk_tokens, max_bins, delta_group, nsub, payload_bytes)
    return head + bytes(HEADER_BYTES - len(head))


def read_header(blob) -> dict:
    """Validates magic, version and sizes; raises ValueError on anything inconsistent."""
    if len(blob) < HEADER_BYTES:
        raise ValueError("wire container: shorter than its header")
    magic, version, flags, L, T, H, D, S, max_bins, delta_group, nsub, payload_bytes = \
        HEADER.unpack_from(bytes(blob[:HEADER.size]))
    if magic != MAGIC:
        raise ValueError("wire container: bad magic %r" % magic)
    if version != VERSION:
        raise ValueError("wire container: version %d is not supported (this reader: %d)" % (version, VERSION))
    if flags & ~FLAG_BF16_MAXIMA:
        raise ValueError("wire container: unknown flags 0x%x" % flags)
    geo = geometry(L, T, H, D, S, max_bins, payload_bytes)
    if geo["nsub"][0] != nsub:
        raise ValueError("wire container: %d sub-chunks recorded, geometry gives %d" % (nsub, geo["nsub"][0]))
    if len(blob) != geo["total"][0]:
        raise ValueError("wire container: %d bytes, geometry gives %d" % (len(blob), geo["total"][0]))
    if payload_bytes > nsub * 2 * L * H * D * MAX_STREAM_BYTES:
        raise ValueError("wire container: payload larger than 256 bytes per stream")
    return dict(num_layers=L, num_tokens=T, num_heads=H, head_size=D, chunk_tokens=S, max_bins=max_bins,
                delta_group=delta_group, nsub=nsub, payload_bytes=payload_bytes,
                bf16_maxima=bool(flags & FLAG_BF16_MAXIMA), geometry=geo)


# --------------------------------------------------------------------------- #
# host form (numpy): the definition of the format, used by the CPU tests
# --------------------------------------------------------------------------- #
def pack_host(cdf: np.ndarray, maxima_bits: np.ndarray, lengths: np.ndarray, payload: np.ndarray,
              num_heads: int, head_size: int, chunk_tokens: int, delta_group: int = 0,
              bf16_maxima: bool = False) -> bytes:
    """cdf int16/uint16 [nchunks, 2L, C, Lp]; maxima_bits uint16 [2, L, T]; lengths int32
    [nsub, 2L, C]; payload uint8 [n]."""
    nchunks, rows, C, lp = cdf.shape
    L, T = maxima_bits.shape[1:]
    if rows != 2 * L or C != num_heads * head_size or lengths.shape[1:] != (rows, C):
        raise ValueError("wire container: array shapes do not agree")
    geo = geometry(L, T, num_heads, head_size, chunk_tokens, lp - 1, payload.size)
    if geo["nchunks"][0] != nchunks or geo["nsub"][0] != lengths.shape[0]:
        raise ValueError("wire container: chunk counts do not agree with the token count")
    if int(np.minimum(lengths, MAX_STREAM_BYTES).astype(np.int64).sum()) != payload.size:
        raise ValueError("wire container: payload size is not the sum of the stream lengths")
    buf = bytearray(geo["total"][0])
    buf[:HEADER_BYTES] = write_header(L, T, num_heads, head_size, chunk_tokens, lp - 1, delta_group,
                                      lengths.shape[0], payload.size, bf16_maxima)
    for name, arr, dt in (("cdf", cdf, "<u2"), ("maxima", maxima_bits, "<u2"), ("lengths", lengths, "<i4"),
                          ("payload", payload, "u1")):
        off, size = geo[name]
        a = np.ascontiguousarray(arr)
        if a.dtype == np.int16:
            a = a.view(np.uint16)
        raw = a.astype(dt, copy=False).tobytes()
        assert len(raw) == size
        buf[off:off + size] = raw
    return bytes(buf)


def unpack_host(blob):
    """-> (header dict, cdf uint16 [nchunks, 2L, C, Lp], maxima uint16 [2, L, T], lengths int32
    [nsub, 2L, C], payload uint8 [n]) as read-only numpy views of the blob."""
    h = read_header(blob)
    geo = h["geometry"]
    L, T, C = h["num_layers"], h["num_tokens"], h["num_heads"] * h["head_size"]
    mv = memoryview(blob)

    def section(name, dt, shape):
        off, size = geo[name]
        return np.frombuffer(mv[off:off + size], dtype=dt).reshape(shape)
    cdf = section("cdf", "<u2", (geo["nchunks"][0], 2 * L, C, h["max_bins"] + 1))
    maxima = section("maxima", "<u2", (2, L, T))
    lengths = section("lengths", "<i4", (h["nsub"], 2 * L, C))
    payload = section("payload", "u1", (h["payload_bytes"],))
    if int(np.minimum(lengths, MAX_STREAM_BYTES).astype(np.int64).sum()) != h["payload_bytes"] \
            or (lengths.size and int(lengths.min()) < 0):
        raise ValueError("wire container: payload size is not the sum of the stream lengths")
    return h, cdf, maxima, lengths, payload


# --------------------------------------------------------------------------- #
# device form: one staging buffer, one copy over PCIe per direction
# --------------------------------------------------------------------------- #
def pack_chunks(enc, first_chunk: int = 0, num_chunks: Optional[int] = None, per_chunk: bool = True) -> List[bytes]:
    """Blobs for chunks [first_chunk, first_chunk + num_chunks) of an `EncodedKV`: one blob per
    chunk (what one `to_bytes` call of the reference covers) or, with per_chunk=False, a single
    blob holding all of them.  All blobs are assembled in one device buffer and leave the GPU
    in one copy into pinned host memory."""
    import torch
    nch = enc.num_chunks
    if num_chunks is None:
        num_chunks = nch - first_chunk
    if first_chunk < 0 or num_chunks <= 0 or first_chunk + num_chunks > nch:
        raise ValueError("chunk range outside the encoded tensor")
    enc.check()
    L, H, D, S, T = enc.num_layers, enc.num_heads, enc.head_size, enc.chunk_tokens, enc.num_tokens
    spc = enc.subchunks_per_chunk
    bounds = enc.sub_boundaries()
    bf16 = enc.maxima.dtype == torch.bfloat16
    groups = [(c, c + 1) for c in range(first_chunk, first_chunk + num_chunks)] if per_chunk \
        else [(first_chunk, first_chunk + num_chunks)]
    plans, total = [], 0
    for c0, c1 in groups:
        t0, t1 = c0 * S, min(c1 * S, T)
        g0, g1 = c0 * spc, min(c1 * spc, enc.lengths.shape[0])
        nbytes = bounds[g1] - bounds[g0]
        table_tokens = min(S, t1 - t0)          # a short last chunk is a blob of its own length
        geo = geometry(L, t1 - t0, H, D, table_tokens, enc.max_bins, nbytes)
        head = write_header(L, t1 - t0, H, D, table_tokens, enc.max_bins, enc.delta_group, g1 - g0, nbytes, bf16)
        plans.append((total, geo, head, (c0, c1, t0, t1, g0, g1)))
        total += geo["total"][0]
    dev = enc.payload.device
    stage = torch.zeros(total, dtype=torch.uint8, device=dev)
    heads = torch.frombuffer(bytearray(b"".join(p[2] for p in plans)), dtype=torch.uint8).to(dev)
    for i, (base, geo, head, (c0, c1, t0, t1, g0, g1)) in enumerate(plans):
        stage[base:base + HEADER_BYTES] = heads[i * HEADER_BYTES:(i + 1) * HEADER_BYTES]
        for name, src in (("cdf", enc.cdf[c0:c1]), ("maxima", enc.maxima[:, :, t0:t1]),
                          ("lengths", enc.lengths[g0:g1]), ("payload", enc.payload[bounds[g0]:bounds[g1]])):
            off, size = geo[name]
            if size:
                stage[base + off:base + off + size].view(src.dtype).view(src.shape).copy_(src)
    host = torch.empty(total, dtype=torch.uint8, pin_memory=True)
    host.copy_(stage, non_blocking=False)
    raw = host.numpy()
    return [raw[base:base + geo["total"][0]].tobytes() for base, geo, _, _ in plans]


def unpack_to_device(blob, device):
    """-> (header dict, cdf, maxima, lengths, payload) as views of one device buffer that the
    blob reached in a single copy from pinned host memory."""
    import torch
    h = read_header(blob)
    geo = h["geometry"]
    L, T, C = h["num_layers"], h["num_tokens"], h["num_heads"] * h["head_size"]
    host = torch.empty(len(blob), dtype=torch.uint8, pin_memory=True)
    host.numpy()[:] = np.frombuffer(blob, dtype=np.uint8)
    buf = host.to(device, non_blocking=False)

    def section(name, dtype, shape):
        off, size = geo[name]
        return buf[off:off + size].view(dtype).view(shape)
    cdf = section("cdf", torch.int16, (geo["nchunks"][0], 2 * L, C, h["max_bins"] + 1))
    maxima = section("maxima", torch.bfloat16 if h["bf16_maxima"] else torch.float16, (2, L, T))
    lengths = section("lengths", torch.int32, (h["nsub"], 2 * L, C))
    payload = section("payload", torch.uint8, (h["payload_bytes"],))
    return h, cdf, maxima, lengths, payload
