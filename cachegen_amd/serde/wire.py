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

Version 2 ("compact") stores the same information in fewer bytes, for chunks of at most 256
tokens, where the 66-byte table per 256-symbol stream outweighs the payload:

    tables   nsym uint8 [nchunks, 2L]: symbols that occur in a (chunk, row), then for every
             (chunk, row, channel) the first nsym histogram counts as one byte each
    lengths  uint16 when every length fits

A table is a function of its histogram (cal_cdf.cu:29-49: cdf[i] = (0xFFFF - max_bins) *
cum[i] / n + i), and for n <= 256 tokens the histogram is recovered from the table exactly
(the scale exceeds n, so distinct running sums give distinct quotients); the writer checks that
the rebuilt tables equal the originals and keeps the raw tables otherwise.  A count of 256
(one symbol for a whole chunk) is stored as 255; the reader adds what is missing from the
chunk's token count back to that entry.
"""
import struct
from typing import Dict, List, Optional, Tuple

import numpy as np

MAGIC = b"CGKV"
VERSION = 1
VERSION_COMPACT = 2
ALIGN = 64
HEADER_BYTES = 64
# magic, version, flags, L, T, H, D, chunk_tokens, max_bins, delta_group, nsub, payload_bytes,
# tables_bytes (version 2 only; zero in version 1)
HEADER = struct.Struct("<4sHHIIIIIIIIQQ")
FLAG_BF16_MAXIMA = 1
FLAG_COUNT_TABLES = 2        # version 2: tables stored as histogram counts
FLAG_LENGTHS_U16 = 4         # version 2: lengths stored as uint16
MAX_STREAM_BYTES = 256


def _up(n: int) -> int:
    return (n + ALIGN - 1) // ALIGN * ALIGN


def is_flat(blob) -> bool:
    return len(blob) >= 4 and bytes(blob[:4]) == MAGIC


def geometry(num_layers: int, num_tokens: int, num_heads: int, head_size: int, chunk_tokens: int,
             max_bins: int, payload_bytes: int, tables_bytes: Optional[int] = None,
             lengths_itemsize: int = 4) -> Dict[str, Tuple[int, int]]:
    """Section name -> (byte offset, byte size), plus "total" -> (size of the blob, 0).
    tables_bytes: size of the table section when it does not hold raw tables."""
    if min(num_layers, num_tokens, num_heads, head_size, chunk_tokens, max_bins) <= 0 or payload_bytes < 0:
        raise ValueError("wire container: sizes must be positive")
    C = num_heads * head_size
    nchunks = -(-num_tokens // chunk_tokens)
    full, rest = divmod(num_tokens, chunk_tokens)
    nsub = full * (-(-chunk_tokens // MAX_STREAM_BYTES)) + (-(-rest // MAX_STREAM_BYTES))
    raw_tables = nchunks * 2 * num_layers * C * (max_bins + 1) * 2
    sizes = [("cdf", raw_tables if tables_bytes is None else tables_bytes),
             ("maxima", 2 * num_layers * num_tokens * 2),
             ("lengths", nsub * 2 * num_layers * C * lengths_itemsize),
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
                 nsub, payload_bytes, bf16_maxima, version=VERSION, extra_flags=0, tables_bytes=0) -> bytes:
    flags = (FLAG_BF16_MAXIMA if bf16_maxima else 0) | extra_flags
    head = HEADER.pack(MAGIC, version, flags, num_layers, num_tokens, num_heads, head_size, chunk_tokens,
                       max_bins, delta_group, nsub, payload_bytes, tables_bytes)
    return head + bytes(HEADER_BYTES - len(head))


def read_header(blob) -> dict:
    """Validates magic, version and sizes; raises ValueError on anything inconsistent."""
    if len(blob) < HEADER_BYTES:
        raise ValueError("wire container: shorter than its header")
    magic, version, flags, L, T, H, D, S, max_bins, delta_group, nsub, payload_bytes, tables_bytes = \
        HEADER.unpack_from(bytes(blob[:HEADER.size]))
    if magic != MAGIC:
        raise ValueError("wire container: bad magic %r" % magic)
    if version not in (VERSION, VERSION_COMPACT):
        raise ValueError("wire container: version %d is not supported (this reader: up to %d)"
                         % (version, VERSION_COMPACT))
    known = FLAG_BF16_MAXIMA if version == VERSION else FLAG_BF16_MAXIMA | FLAG_COUNT_TABLES | FLAG_LENGTHS_U16
    if flags & ~known:
        raise ValueError("wire container: unknown flags 0x%x" % flags)
    count_tables = bool(flags & FLAG_COUNT_TABLES)
    if count_tables and S > MAX_STREAM_BYTES:
        raise ValueError("wire container: count tables need chunks of at most 256 tokens")
    geo = geometry(L, T, H, D, S, max_bins, payload_bytes, tables_bytes if count_tables else None,
                   2 if flags & FLAG_LENGTHS_U16 else 4)
    if geo["nsub"][0] != nsub:
        raise ValueError("wire container: %d sub-chunks recorded, geometry gives %d" % (nsub, geo["nsub"][0]))
    if len(blob) != geo["total"][0]:
        raise ValueError("wire container: %d bytes, geometry gives %d" % (len(blob), geo["total"][0]))
    if payload_bytes > nsub * 2 * L * H * D * MAX_STREAM_BYTES:
        raise ValueError("wire container: payload larger than 256 bytes per stream")
    return dict(num_layers=L, num_tokens=T, num_heads=H, head_size=D, chunk_tokens=S, max_bins=max_bins,
                delta_group=delta_group, nsub=nsub, payload_bytes=payload_bytes,
                bf16_maxima=bool(flags & FLAG_BF16_MAXIMA), count_tables=count_tables,
                lengths_u16=bool(flags & FLAG_LENGTHS_U16), version=version, geometry=geo)


# --------------------------------------------------------------------------- #
# tables <-> histogram counts (numpy: the definition; the device code below mirrors it)
# --------------------------------------------------------------------------- #
def chunk_token_counts(num_tokens: int, chunk_tokens: int) -> List[int]:
    return [min(chunk_tokens, num_tokens - t0) for t0 in range(0, num_tokens, chunk_tokens)]


def tables_to_counts(cdf: np.ndarray, tokens: List[int]) -> Optional[np.ndarray]:
    """cdf uint16 [nchunks, 2L, C, Lp] built over tokens[chunk] <= 256 tokens each ->
    histogram counts int64 [nchunks, 2L, C, Lp - 1], or None if the tables are not exactly what
    cal_cdf.cu:29-49 gives for some histogram."""
    lp = cdf.shape[-1]
    scale = 0xFFFF - (lp - 1)
    n = np.asarray(tokens, dtype=np.int64).reshape(-1, 1, 1, 1)
    q = cdf.astype(np.int64) - np.arange(lp, dtype=np.int64)
    cum = (q * n + scale - 1) // scale
    counts = np.diff(cum, axis=-1)
    if (cum[..., 0] != 0).any() or (counts < 0).any() or not np.array_equal(counts_to_tables(counts, tokens), cdf):
        return None
    return counts


def counts_to_tables(counts: np.ndarray, tokens: List[int]) -> np.ndarray:
    """The inverse: cdf[i] = (0xFFFF - max_bins) * cum[i] / n + i in integers."""
    lp = counts.shape[-1] + 1
    scale = 0xFFFF - (lp - 1)
    n = np.asarray(tokens, dtype=np.int64).reshape(-1, 1, 1, 1)
    cum = np.concatenate([np.zeros(counts.shape[:-1] + (1,), dtype=np.int64), np.cumsum(counts, axis=-1)], axis=-1)
    return ((scale * cum) // n + np.arange(lp, dtype=np.int64)).astype(np.uint16)


def pack_counts(counts: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """-> (nsym uint8 [nchunks, 2L], bytes uint8 [sum of C * nsym]): per (chunk, row) the number
    of leading symbols that hold every occurrence, then those counts, clamped to 255, for each
    channel in turn."""
    used = counts.sum(axis=2) > 0                                    # [nchunks, 2L, nsyms]
    nsyms = counts.shape[-1]
    nsym = np.where(used.any(-1), nsyms - np.argmax(used[..., ::-1], axis=-1), 1).astype(np.uint8)
    mask = np.arange(nsyms)[None, None, None, :] < nsym[:, :, None, None].astype(np.int64)
    mask = np.broadcast_to(mask, counts.shape)
    return nsym, np.minimum(counts, 255).astype(np.uint8)[mask]


def unpack_counts(nsym: np.ndarray, data: np.ndarray, C: int, nsyms: int, tokens: List[int]) -> np.ndarray:
    mask = np.arange(nsyms)[None, None, None, :] < nsym[:, :, None, None].astype(np.int64)
    mask = np.broadcast_to(mask, nsym.shape + (C, nsyms))
    if int(mask.sum()) != data.size:
        raise ValueError("wire container: table section does not match its symbol counts")
    counts = np.zeros(mask.shape, dtype=np.int64)
    counts[mask] = data
    n = np.asarray(tokens, dtype=np.int64).reshape(-1, 1, 1)
    missing = n - counts.sum(-1)                                     # 1 where a count of 256 was clamped
    if ((missing != 0) & ~((missing == 1) & ((counts == 255).sum(-1) == 1))).any():
        raise ValueError("wire container: histogram counts do not add up to the chunk's tokens")
    return counts + (counts == 255) * missing[..., None]


# --------------------------------------------------------------------------- #
# host form (numpy): the definition of the format, used by the CPU tests
# --------------------------------------------------------------------------- #
def pack_host(cdf: np.ndarray, maxima_bits: np.ndarray, lengths: np.ndarray, payload: np.ndarray,
              num_heads: int, head_size: int, chunk_tokens: int, delta_group: int = 0,
              bf16_maxima: bool = False, compact: bool = False) -> bytes:
    """cdf int16/uint16 [nchunks, 2L, C, Lp]; maxima_bits uint16 [2, L, T]; lengths int32
    [nsub, 2L, C]; payload uint8 [n].  compact: write version 2."""
    nchunks, rows, C, lp = cdf.shape
    L, T = maxima_bits.shape[1:]
    if rows != 2 * L or C != num_heads * head_size or lengths.shape[1:] != (rows, C):
        raise ValueError("wire container: array shapes do not agree")
    cdf = np.ascontiguousarray(cdf)
    if cdf.dtype == np.int16:
        cdf = cdf.view(np.uint16)
    version, flags, tables, lengths_out = VERSION, 0, cdf.astype("<u2", copy=False).tobytes(), lengths.astype("<i4")
    tables_bytes = None
    if compact:
        version = VERSION_COMPACT
        counts = tables_to_counts(cdf, chunk_token_counts(T, chunk_tokens)) if chunk_tokens <= MAX_STREAM_BYTES else None
        if counts is not None:
            nsym, data = pack_counts(counts)
            tables = nsym.tobytes() + data.tobytes()
            tables_bytes = len(tables)
            flags |= FLAG_COUNT_TABLES
        if lengths.size == 0 or (int(lengths.min()) >= 0 and int(lengths.max()) <= 0xFFFF):
            lengths_out = lengths.astype("<u2")
            flags |= FLAG_LENGTHS_U16
    geo = geometry(L, T, num_heads, head_size, chunk_tokens, lp - 1, payload.size, tables_bytes,
                   lengths_out.dtype.itemsize)
    if geo["nchunks"][0] != nchunks or geo["nsub"][0] != lengths.shape[0]:
        raise ValueError("wire container: chunk counts do not agree with the token count")
    if int(np.minimum(lengths, MAX_STREAM_BYTES).astype(np.int64).sum()) != payload.size:
        raise ValueError("wire container: payload size is not the sum of the stream lengths")
    buf = bytearray(geo["total"][0])
    buf[:HEADER_BYTES] = write_header(L, T, num_heads, head_size, chunk_tokens, lp - 1, delta_group,
                                      lengths.shape[0], payload.size, bf16_maxima, version, flags,
                                      tables_bytes or 0)
    for name, raw in (("cdf", tables), ("maxima", np.ascontiguousarray(maxima_bits).astype("<u2", copy=False).tobytes()),
                      ("lengths", np.ascontiguousarray(lengths_out).tobytes()),
                      ("payload", np.ascontiguousarray(payload).tobytes())):
        off, size = geo[name]
        assert len(raw) == size
        buf[off:off + size] = raw
    return bytes(buf)


def unpack_host(blob):
    """-> (header dict, cdf uint16 [nchunks, 2L, C, Lp], maxima uint16 [2, L, T], lengths int32
    [nsub, 2L, C], payload uint8 [n]): read-only numpy views of the blob where the stored form is
    the array itself, new arrays where it is not (version 2)."""
    h = read_header(blob)
    geo = h["geometry"]
    L, T, C = h["num_layers"], h["num_tokens"], h["num_heads"] * h["head_size"]
    lp, nchunks = h["max_bins"] + 1, geo["nchunks"][0]
    mv = memoryview(blob)

    def section(name, dt, shape):
        off, size = geo[name]
        return np.frombuffer(mv[off:off + size], dtype=dt).reshape(shape)
    if h["count_tables"]:
        raw = section("cdf", "u1", (-1,))
        if raw.size < nchunks * 2 * L:
            raise ValueError("wire container: table section does not match its symbol counts")
        nsym = raw[:nchunks * 2 * L].reshape(nchunks, 2 * L)
        if int(nsym.min()) < 1 or int(nsym.max()) > lp - 1:
            raise ValueError("wire container: symbol count outside the table")
        tokens = chunk_token_counts(T, h["chunk_tokens"])
        cdf = counts_to_tables(unpack_counts(nsym, raw[nchunks * 2 * L:], C, lp - 1, tokens), tokens)
    else:
        cdf = section("cdf", "<u2", (nchunks, 2 * L, C, lp))
    maxima = section("maxima", "<u2", (2, L, T))
    lengths = section("lengths", "<u2" if h["lengths_u16"] else "<i4", (h["nsub"], 2 * L, C)).astype(np.int32, copy=False)
    payload = section("payload", "u1", (h["payload_bytes"],))
    if int(np.minimum(lengths, MAX_STREAM_BYTES).astype(np.int64).sum()) != h["payload_bytes"] \
            or (lengths.size and int(lengths.min()) < 0):
        raise ValueError("wire container: payload size is not the sum of the stream lengths")
    return h, cdf, maxima, lengths, payload


# --------------------------------------------------------------------------- #
# device form: one staging buffer, one copy over PCIe per direction
# --------------------------------------------------------------------------- #
def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _device_counts_launch(cdf, tokens):
    """First half of the device form of tables_to_counts + pack_counts for cdf int16
    [nchunks, 2L, C, Lp]: launches the conversion and returns (dense counts uint8 [G, C, Lp-1],
    nsym int32 [G], inexact int32 [1]), all still on the device and not waited for."""
    import torch
    from .. import _lib
    nchunks, rows, C, lp = cdf.shape
    G = nchunks * rows
    dev = cdf.device
    cdf = cdf.contiguous()
    tok = torch.tensor([t for t in tokens for _ in range(rows)], dtype=torch.int32).to(dev, non_blocking=True)
    dense = torch.empty((G, C, lp - 1), dtype=torch.uint8, device=dev)
    nsym = torch.empty(G, dtype=torch.int32, device=dev)
    inexact = torch.empty(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().cg_tables_to_counts(cdf.data_ptr(), lp - 1, G, C, tok.data_ptr(), dense.data_ptr(),
                                                  nsym.data_ptr(), inexact.data_ptr(), _stream()))
    return dense, nsym, inexact


def _device_counts_finish(dense, nsym, ks):
    """Second half: ks is nsym read back on the host; returns the ragged count bytes uint8 on
    the device."""
    import torch
    from .. import _lib
    G, C, nb = dense.shape
    dev = dense.device
    starts, total = [], 0
    for k in ks:
        starts.append(total)
        total += C * k
    data = torch.empty(total, dtype=torch.uint8, device=dev)
    d_starts = torch.tensor(starts, dtype=torch.int64).to(dev, non_blocking=True)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().cg_pack_counts(dense.data_ptr(), nb, G, C, nsym.data_ptr(), d_starts.data_ptr(),
                                             data.data_ptr(), _stream()))
    return data


def _device_counts(cdf, tokens):
    """Device form of tables_to_counts + pack_counts for cdf int16 [nchunks, 2L, C, Lp]:
    (nsym list per (chunk, row), ragged count bytes uint8 on the device) or None if some table is
    not the table of a histogram."""
    import torch
    dense, nsym, inexact = _device_counts_launch(cdf, tokens)
    host = torch.cat([nsym, inexact]).tolist()
    if host[-1]:
        return None
    return host[:-1], _device_counts_finish(dense, nsym, host[:-1])


def _raise_if_invalid_counts(invalid):
    if int(invalid.item()):
        raise ValueError("wire container: histogram counts do not add up to the chunk's tokens")


def _device_tables(nsym_host, nsym_dev, data, C, lp, tokens, defer=False):
    """Device form of unpack_counts + counts_to_tables -> cdf int16 [nchunks, 2L, C, Lp].
    nsym_host: numpy uint8 [nchunks, 2L] (read from the blob on the host), nsym_dev the same bytes
    on the device.  defer: do not wait for the kernel's verdict on the counts; returns
    (cdf, check) where check() waits and raises."""
    import torch
    from .. import _lib
    nchunks, rows = nsym_host.shape
    G = nchunks * rows
    dev = data.device
    sizes = nsym_host.astype(np.int64).ravel() * C
    starts = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int64)
    if int(sizes.sum()) != data.numel():
        raise ValueError("wire container: table section does not match its symbol counts")
    small = torch.from_numpy(np.concatenate([starts, np.repeat(np.asarray(tokens, dtype=np.int64), rows)])).to(dev)
    tok = small[G:].to(torch.int32)
    cdf = torch.empty((nchunks, rows, C, lp), dtype=torch.int16, device=dev)
    invalid = torch.empty(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().cg_counts_to_tables(data.data_ptr(), data.numel(), lp - 1, G, C, tok.data_ptr(),
                                                  nsym_dev.data_ptr(), small.data_ptr(), cdf.data_ptr(),
                                                  invalid.data_ptr(), _stream()))
    if defer:
        return cdf, (lambda: _raise_if_invalid_counts(invalid))
    _raise_if_invalid_counts(invalid)
    return cdf


def pack_chunks(enc, first_chunk: int = 0, num_chunks: Optional[int] = None, per_chunk: bool = True,
                compact: bool = False) -> List[bytes]:
    """Blobs for chunks [first_chunk, first_chunk + num_chunks) of an `EncodedKV`: one blob per
    chunk (what one `to_bytes` call of the reference covers) or, with per_chunk=False, a single
    blob holding all of them; compact: version 2.  All blobs are assembled in one device buffer
    and leave the GPU in one copy into pinned host memory."""
    import torch
    nch = enc.num_chunks
    if num_chunks is None:
        num_chunks = nch - first_chunk
    if first_chunk < 0 or num_chunks <= 0 or first_chunk + num_chunks > nch:
        raise ValueError("chunk range outside the encoded tensor")
    L, H, D, S, T = enc.num_layers, enc.num_heads, enc.head_size, enc.chunk_tokens, enc.num_tokens
    C = H * D
    spc = enc.subchunks_per_chunk
    bf16 = enc.maxima.dtype == torch.bfloat16
    groups = [(c, c + 1) for c in range(first_chunk, first_chunk + num_chunks)] if per_chunk \
        else [(first_chunk, first_chunk + num_chunks)]
    all_tokens = chunk_token_counts(T, S)
    c0, c1 = first_chunk, first_chunk + num_chunks

    # everything the host has to know before it can lay the blobs out, read back at once:
    # status word, payload offset at every sub-chunk boundary, smallest and largest stream
    # length, and (compact) the symbol count of every table plus the flag that says whether
    # all tables are tables of histograms
    dev = enc.payload.device
    nsub = enc.lengths.shape[0]
    idx = torch.arange(0, nsub + 1, device=dev) * (2 * L * C)
    want_counts = compact and S <= MAX_STREAM_BYTES
    parts = [enc.status.to(torch.int64).reshape(1), enc.offsets[idx]]
    if compact:
        parts += [enc.lengths.min().to(torch.int64).reshape(1), enc.lengths.max().to(torch.int64).reshape(1)]
    if want_counts:
        dense, nsym_dev, inexact = _device_counts_launch(enc.cdf[c0:c1], all_tokens[c0:c1])
        parts += [inexact.to(torch.int64), nsym_dev.to(torch.int64)]
    meta = torch.cat(parts).tolist()
    enc.raise_for_status(meta[0])
    bounds = meta[1:nsub + 2]
    rest = meta[nsub + 2:]

    version, flags, lengths_src = VERSION, 0, enc.lengths
    packed = None                       # (nsym [nch, 2L], data, byte offset of every (chunk, row) in data)
    if compact:
        version = VERSION_COMPACT
        lo, hi = rest[0], rest[1]
        if want_counts and not rest[2]:
            ks = rest[3:]                                        # nsym per (chunk, row)
            data = _device_counts_finish(dense, nsym_dev, ks)    # ragged count bytes
            starts = [0]
            for k in range(c1 - c0):
                starts.append(starts[-1] + C * sum(ks[k * 2 * L:(k + 1) * 2 * L]))
            nsym = nsym_dev.to(torch.uint8).view(c1 - c0, 2 * L)
            packed = (nsym, data, starts)
            flags |= FLAG_COUNT_TABLES
        if lo >= 0 and hi <= 0xFFFF:
            lengths_src = enc.lengths.to(torch.int16)         # bit pattern of the uint16 value
            flags |= FLAG_LENGTHS_U16

    plans, total = [], 0
    for c0, c1 in groups:
        t0, t1 = c0 * S, min(c1 * S, T)
        g0, g1 = c0 * spc, min(c1 * spc, enc.lengths.shape[0])
        nbytes = bounds[g1] - bounds[g0]
        table_tokens = min(S, t1 - t0)          # a short last chunk is a blob of its own length
        tables_bytes = None
        if packed is not None:
            k0, k1 = c0 - first_chunk, c1 - first_chunk
            tables_bytes = (k1 - k0) * 2 * L + packed[2][k1] - packed[2][k0]
        geo = geometry(L, t1 - t0, H, D, table_tokens, enc.max_bins, nbytes, tables_bytes,
                       lengths_src.element_size())
        head = write_header(L, t1 - t0, H, D, table_tokens, enc.max_bins, enc.delta_group, g1 - g0, nbytes, bf16,
                            version, flags, tables_bytes or 0)
        plans.append((total, geo, head, (c0, c1, t0, t1, g0, g1)))
        total += geo["total"][0]
    stage = torch.zeros(total, dtype=torch.uint8, device=dev)
    heads = torch.frombuffer(bytearray(b"".join(p[2] for p in plans)), dtype=torch.uint8).to(dev)

    def place(base, span, src):
        off, size = span
        if size:
            stage[base + off:base + off + size].view(src.dtype).view(src.shape).copy_(src)
    for i, (base, geo, head, (c0, c1, t0, t1, g0, g1)) in enumerate(plans):
        stage[base:base + HEADER_BYTES] = heads[i * HEADER_BYTES:(i + 1) * HEADER_BYTES]
        if packed is None:
            place(base, geo["cdf"], enc.cdf[c0:c1])
        else:
            k0, k1 = c0 - first_chunk, c1 - first_chunk
            off, size = geo["cdf"]
            head_bytes = (k1 - k0) * 2 * L
            place(base, (off, head_bytes), packed[0][k0:k1])
            place(base, (off + head_bytes, size - head_bytes), packed[1][packed[2][k0]:packed[2][k1]])
        place(base, geo["maxima"], enc.maxima[:, :, t0:t1])
        place(base, geo["lengths"], lengths_src[g0:g1])
        place(base, geo["payload"], enc.payload[bounds[g0]:bounds[g1]])
    host = torch.empty(total, dtype=torch.uint8, pin_memory=True)
    host.copy_(stage, non_blocking=False)
    raw = host.numpy()
    return [raw[base:base + geo["total"][0]].tobytes() for base, geo, _, _ in plans]


def unpack_to_device(blob, device, defer_checks=False):
    """-> (header dict, cdf, maxima, lengths, payload) on the device, which the blob reached in a
    single copy from pinned host memory: views of that buffer where the stored form is the
    tensor itself, rebuilt tensors where it is not (version 2).  The stream lengths are checked
    against the payload size on the host.  defer_checks: nothing here waits for the device; the
    header dict then holds "check", to be called once the caller has queued its own work: it
    waits for the device and raises what the device-side checks found."""
    import torch
    h = read_header(blob)
    geo = h["geometry"]
    L, T, C = h["num_layers"], h["num_tokens"], h["num_heads"] * h["head_size"]
    lp, nchunks = h["max_bins"] + 1, geo["nchunks"][0]
    host = torch.empty(len(blob), dtype=torch.uint8, pin_memory=True)
    host.numpy()[:] = np.frombuffer(blob, dtype=np.uint8)
    buf = host.to(device, non_blocking=False)      # waits: the pinned buffer is free for the next call at once
    # the lengths are in the blob: their sum is checked here, without asking the device
    off, size = geo["lengths"]
    host_lengths = np.frombuffer(blob, dtype=np.uint16 if h["lengths_u16"] else np.int32, count=h["nsub"] * 2 * L * C,
                                 offset=off)
    # one rule everywhere: a stream occupies min(length, 256) bytes of the payload
    if int(np.minimum(host_lengths, MAX_STREAM_BYTES).sum(dtype=np.int64)) != h["payload_bytes"] \
            or (host_lengths.size and int(host_lengths.min()) < 0):
        raise ValueError("wire container: payload size is not the sum of the stream lengths")
    h["check"] = lambda: None

    def section(name, dtype, shape):
        off, size = geo[name]
        return buf[off:off + size].view(dtype).view(shape)
    if h["count_tables"]:
        raw = section("cdf", torch.uint8, (-1,))
        if raw.numel() < nchunks * 2 * L:
            raise ValueError("wire container: table section does not match its symbol counts")
        off = geo["cdf"][0]
        nsym_host = np.frombuffer(blob, dtype=np.uint8, count=nchunks * 2 * L, offset=off).reshape(nchunks, 2 * L)
        if int(nsym_host.min()) < 1 or int(nsym_host.max()) > lp - 1:
            raise ValueError("wire container: symbol count outside the table")
        cdf = _device_tables(nsym_host, raw[:nchunks * 2 * L], raw[nchunks * 2 * L:], C, lp,
                             chunk_token_counts(T, h["chunk_tokens"]), defer=defer_checks)
        if defer_checks:
            cdf, h["check"] = cdf
    else:
        cdf = section("cdf", torch.int16, (nchunks, 2 * L, C, lp))
    maxima = section("maxima", torch.bfloat16 if h["bf16_maxima"] else torch.float16, (2, L, T))
    if h["lengths_u16"]:
        lengths = section("lengths", torch.int16, (h["nsub"], 2 * L, C)).to(torch.int32) & 0xFFFF
    else:
        lengths = section("lengths", torch.int32, (h["nsub"], 2 * L, C))
    payload = section("payload", torch.uint8, (h["payload_bytes"],))
    return h, cdf, maxima, lengths, payload
