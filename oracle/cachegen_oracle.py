"""numpy front end of the CPU oracle (oracle/cachegen_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py as the checker.  The product package never
imports it.

16-bit floats travel as their uint16 bit patterns (numpy has no bfloat16).
`encode_function` / `decode_function` restate the orchestration of
LMCache/lmcache/storage_backend/serde/cachegen_encoder.py:247-301 and
cachegen_decoder.py:77-112,144-173 on top of the C functions.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcachegen_oracle.so")

DT_F16 = 0
DT_BF16 = 1
MAX_TOKENS_PER_STREAM = 256      # cachegen_basics.py:8

_lib = None


def build(force=False):
    """Compile the C restatement with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libcachegen_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.cgo_encode_stream.restype = ctypes.c_int
        _lib.cgo_collect_bytes.restype = ctypes.c_int64
        _lib.cgo_half_to_float.restype = ctypes.c_float
        _lib.cgo_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.cgo_bf16_to_float.restype = ctypes.c_float
        _lib.cgo_bf16_to_float.argtypes = [ctypes.c_uint16]
        _lib.cgo_float_to_half.restype = ctypes.c_uint16
        _lib.cgo_float_to_half.argtypes = [ctypes.c_float]
        _lib.cgo_float_to_bf16.restype = ctypes.c_uint16
        _lib.cgo_float_to_bf16.argtypes = [ctypes.c_float]
        _lib.cgo_max_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def set_threads(n):
    lib().cgo_set_threads(ctypes.c_int(int(n)))


def max_threads():
    return int(lib().cgo_max_threads())


def _estrides(a):
    assert all(s % a.itemsize == 0 for s in a.strides)
    return [s // a.itemsize for s in a.strides]


def quantize(x_bits, bins, dt=DT_F16):
    """x_bits uint16 [nl, nt, nc] (last dim contiguous) -> (sym uint8, max uint16 [nl, nt])."""
    assert x_bits.dtype == np.uint16 and x_bits.ndim == 3
    nl, nt, nc = x_bits.shape
    s = _estrides(x_bits)
    assert s[2] == 1 or nc == 1
    bins = np.ascontiguousarray(bins, dtype=np.float32)
    assert bins.shape == (nl,)
    sym = np.empty((nl, nt, nc), dtype=np.uint8)
    mx = np.empty((nl, nt), dtype=np.uint16)
    lib().cgo_quantize(_p(x_bits), ctypes.c_int(dt), _i64(nl), _i64(nt), _i64(nc),
                       _i64(s[0]), _i64(s[1]), _p(bins), _p(sym), _p(mx))
    return sym, mx


def dequantize(sym, bins, maxima, max_dt=DT_F16, out_dt=DT_F16):
    """sym uint8 [nl, nt, nc], maxima uint16 [nl, nt] -> uint16 bit patterns [nl, nt, nc]."""
    sym = np.ascontiguousarray(sym, dtype=np.uint8)
    nl, nt, nc = sym.shape
    bins = np.ascontiguousarray(bins, dtype=np.float32)
    maxima = np.ascontiguousarray(maxima, dtype=np.uint16).reshape(nl, nt)
    out = np.empty((nl, nt, nc), dtype=np.uint16)
    lib().cgo_dequantize(_p(sym), _i64(nl), _i64(nt), _i64(nc), _p(bins), _p(maxima),
                         ctypes.c_int(max_dt), _p(out), _i64(nt * nc), _i64(nc),
                         ctypes.c_int(out_dt))
    return out


def quantize_delta(x_bits, bins, group, dt=DT_F16):
    """Delta-against-anchor quantization (no counterpart in the reference; see the C file)."""
    nl, nt, nc = x_bits.shape
    s = _estrides(x_bits)
    bins = np.ascontiguousarray(bins, dtype=np.float32)
    sym = np.empty((nl, nt, nc), dtype=np.uint8)
    mx = np.empty((nl, nt), dtype=np.uint16)
    lib().cgo_quantize_delta(_p(x_bits), ctypes.c_int(dt), _i64(nl), _i64(nt), _i64(nc), _i64(s[0]),
                             _i64(s[1]), _p(bins), ctypes.c_int(group), _p(sym), _p(mx))
    return sym, mx


def dequantize_delta(sym, bins, maxima, group, max_dt=DT_F16, out_dt=DT_F16):
    sym = np.ascontiguousarray(sym, dtype=np.uint8)
    nl, nt, nc = sym.shape
    bins = np.ascontiguousarray(bins, dtype=np.float32)
    maxima = np.ascontiguousarray(maxima, dtype=np.uint16).reshape(nl, nt)
    out = np.empty((nl, nt, nc), dtype=np.uint16)
    lib().cgo_dequantize_delta(_p(sym), _i64(nl), _i64(nt), _i64(nc), _p(bins), _p(maxima),
                               ctypes.c_int(max_dt), ctypes.c_int(group), _p(out), _i64(nt * nc),
                               _i64(nc), ctypes.c_int(out_dt))
    return out


def calculate_cdf(sym, max_bins):
    """sym uint8/int8 [nl, nt, nc] (any strides) -> uint16 [nl, nc, max_bins + 1]."""
    sym = sym.view(np.uint8)
    nl, nt, nc = sym.shape
    s = _estrides(sym)
    cdf = np.empty((nl, nc, max_bins + 1), dtype=np.uint16)
    lib().cgo_calculate_cdf(_p(sym), _i64(nl), _i64(nt), _i64(nc), _i64(s[0]), _i64(s[1]),
                            _i64(s[2]), ctypes.c_int(max_bins), _p(cdf))
    return cdf


def encode_stream(cdf_row, syms, cap=MAX_TOKENS_PER_STREAM):
    """One stream: cdf_row uint16 [lp], syms uint8 [n] -> bytes."""
    cdf_row = np.ascontiguousarray(cdf_row, dtype=np.uint16)
    syms = np.ascontiguousarray(syms, dtype=np.uint8)
    out = np.zeros(cap, dtype=np.uint8)
    n = lib().cgo_encode_stream(_p(cdf_row), ctypes.c_int(len(cdf_row)), _p(syms), _i64(1),
                                ctypes.c_int(len(syms)), _p(out), ctypes.c_int(cap))
    return out[:min(n, cap)].tobytes(), n


def decode_stream(cdf_row, data, n):
    """One stream: bytes -> uint8 [n]."""
    cdf_row = np.ascontiguousarray(cdf_row, dtype=np.uint16)
    buf = np.frombuffer(bytes(data) + b"\0", dtype=np.uint8).copy()
    out = np.zeros(max(n, 1), dtype=np.uint8)
    lib().cgo_decode_stream(_p(cdf_row), ctypes.c_int(len(cdf_row)), _p(buf),
                            ctypes.c_int(len(data)), ctypes.c_int(n), _p(out), _i64(1))
    return out[:n]


def encode_fast_new(cdf, sym, out=None, lengths=None, cap=MAX_TOKENS_PER_STREAM):
    """cdf uint16 [nl, nc, lp]; sym uint8 [nl, nt, nc] (any strides).

    Returns (padded uint8 [nl, nc, cap], lengths int32 [nl, nc]); bytes past a
    stream's length keep whatever `out` held."""
    cdf = np.ascontiguousarray(cdf).view(np.uint16)
    sym = sym.view(np.uint8)
    nl, nt, nc = sym.shape
    assert cdf.shape[:2] == (nl, nc)
    s = _estrides(sym)
    if out is None:
        out = np.zeros((nl, nc, cap), dtype=np.uint8)
    if lengths is None:
        lengths = np.zeros((nl, nc), dtype=np.int32)
    assert out.flags.c_contiguous and lengths.flags.c_contiguous
    lib().cgo_encode_fast_new(_p(cdf), ctypes.c_int(cdf.shape[2]), _p(sym), _i64(nl), _i64(nt),
                              _i64(nc), _i64(s[0]), _i64(s[1]), _i64(s[2]), _p(out),
                              ctypes.c_int(out.shape[2]), _p(lengths))
    return out, lengths


def collect_bytes(padded, lengths):
    padded = np.ascontiguousarray(padded, dtype=np.uint8)
    lengths = np.ascontiguousarray(lengths, dtype=np.int32)
    cap = padded.shape[-1]
    total = int(np.minimum(lengths, cap).astype(np.int64).sum())
    out = np.empty(total, dtype=np.uint8)
    n = lib().cgo_collect_bytes(_p(padded), ctypes.c_int(cap), _p(lengths), _i64(lengths.size), _p(out))
    assert n == total
    return out


def decode_fast_prefsum(cdf, data, prefix, nt, out=None):
    """cdf uint16 [nl, nc, lp]; data uint8 [n]; prefix int64 [nl, nc] inclusive sums."""
    cdf = np.ascontiguousarray(cdf).view(np.uint16)
    nl, nc, lp = cdf.shape
    data = np.ascontiguousarray(data, dtype=np.uint8)
    data = np.concatenate([data, np.zeros(8, dtype=np.uint8)])
    prefix = np.ascontiguousarray(prefix, dtype=np.int64)
    if out is None:
        out = np.zeros((nl, nt, nc), dtype=np.uint8)
    o = _estrides(out)
    lib().cgo_decode_fast_prefsum(_p(cdf), ctypes.c_int(lp), _p(data), _p(prefix), _i64(nl),
                                  _i64(nt), _i64(nc), _p(out), _i64(o[0]), _i64(o[1]), _i64(o[2]))
    return out


def decode_fast_new(cdf, padded, lengths, nt, out=None):
    cdf = np.ascontiguousarray(cdf).view(np.uint16)
    nl, nc, lp = cdf.shape
    padded = np.ascontiguousarray(padded, dtype=np.uint8)
    lengths = np.ascontiguousarray(lengths, dtype=np.int32)
    if out is None:
        out = np.zeros((nl, nt, nc), dtype=np.uint8)
    o = _estrides(out)
    lib().cgo_decode_fast_new(_p(cdf), ctypes.c_int(lp), _p(padded), ctypes.c_int(padded.shape[2]),
                              _p(lengths), _i64(nl), _i64(nt), _i64(nc), _p(out),
                              _i64(o[0]), _i64(o[1]), _i64(o[2]))
    return out


def encode_function(kv_bits, key_bins, value_bins, dt=DT_F16, delta_group=0):
    """One `to_bytes` call (encoder.py:247-301) on kv_bits uint16 [L, 2, T, C].

    Returns a dict with the fields of CacheGenGPUEncoderOutput as numpy arrays:
    cdf uint16 [2L, C, Lp], max_tensors_key / max_tensors_value uint16 [L, T],
    data_chunks = list of (bytestream uint8 [n], lengths int32 [2L, C], ntokens),
    plus the intermediate symbols uint8 [2L, T, C]."""
    nl, two, nt, nc = kv_bits.shape
    assert two == 2
    key_bins = np.asarray(key_bins, dtype=np.float32)
    value_bins = np.asarray(value_bins, dtype=np.float32)
    if delta_group > 0:
        sym_k, max_k = quantize_delta(kv_bits[:, 0], key_bins, delta_group, dt)
        sym_v, max_v = quantize_delta(kv_bits[:, 1], value_bins, delta_group, dt)
    else:
        sym_k, max_k = quantize(kv_bits[:, 0], key_bins, dt)
        sym_v, max_v = quantize(kv_bits[:, 1], value_bins, dt)
    sym = np.concatenate([sym_k, sym_v], axis=0)
    cdf = np.concatenate([calculate_cdf(sym_k, int(key_bins.max())),
                          calculate_cdf(sym_v, int(value_bins.max()))], axis=0)
    chunks = []
    padded = np.zeros((2 * nl, nc, MAX_TOKENS_PER_STREAM), dtype=np.uint8)
    lengths = np.zeros((2 * nl, nc), dtype=np.int32)
    for start in range(0, nt, MAX_TOKENS_PER_STREAM):
        end = min(start + MAX_TOKENS_PER_STREAM, nt)
        encode_fast_new(cdf, sym[:, start:end, :], padded, lengths)
        chunks.append((collect_bytes(padded, lengths), lengths.copy(), end - start))
    return dict(cdf=cdf, max_tensors_key=max_k, max_tensors_value=max_v,
                data_chunks=chunks, symbols=sym)


def decode_function(enc, key_bins, value_bins, max_dt=DT_F16, out_dt=DT_F16, delta_group=0):
    """One `from_bytes` call (decoder.py:144-173) up to the [L, 2, T, C] blob.

    Returns (symbols uint8 [2L, T, C], kv_bits uint16 [L, 2, T, C])."""
    cdf = enc["cdf"]
    nl2, nc, _ = cdf.shape
    nl = nl2 // 2
    nt = enc["max_tensors_key"].shape[1]
    sym = np.zeros((nl2, nt, nc), dtype=np.uint8)
    start = 0
    for data, lengths, n in enc["data_chunks"]:
        prefix = lengths.astype(np.int64).ravel().cumsum().reshape(lengths.shape)
        decode_fast_prefsum(cdf, data, prefix, n, sym[:, start:start + n, :])
        start += n
    if delta_group > 0:
        k = dequantize_delta(sym[:nl], key_bins, enc["max_tensors_key"], delta_group, max_dt, out_dt)
        v = dequantize_delta(sym[nl:], value_bins, enc["max_tensors_value"], delta_group, max_dt, out_dt)
    else:
        k = dequantize(sym[:nl], key_bins, enc["max_tensors_key"], max_dt, out_dt)
        v = dequantize(sym[nl:], value_bins, enc["max_tensors_value"], max_dt, out_dt)
    return sym, np.stack([k, v], axis=1)
