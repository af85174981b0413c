"""Whole-tensor encode / decode of a KV cache: every chunk in a handful of launches.

`encode_kv` does, for all chunks of a KV cache at once, what one `to_bytes` call of
the reference does per chunk (LMCache/lmcache/storage_backend/serde/
cachegen_encoder.py:247-301): quantize, build one table per (chunk, layer, channel),
arithmetic-code one stream per (256-token sub-chunk, layer, channel) and pack the
streams back to back.  `decode_kv` is the inverse up to the dequantized 16-bit
tensor (cachegen_decoder.py:77-112, 144-173).  `EncodedKV.chunk(i)` slices out the
fields the reference's CacheGenGPUEncoderOutput holds for chunk i.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib

MAX_TOKENS_PER_STREAM = 256
_DT = {torch.float16: _lib.DT_F16, torch.bfloat16: _lib.DT_BF16}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _kv_strides(t, fmt):
    """Element strides (layer, k|v, token, head) of a [L,2,T,H,D] ("vllm") or
    [L,2,H,T,D] ("huggingface") tensor whose last dimension is contiguous."""
    if t.dim() != 5 or t.shape[1] != 2:
        raise RuntimeError("expected a KV tensor with 5 dimensions, the second of size 2")
    if t.stride(4) != 1 and t.shape[4] != 1:
        raise RuntimeError("the head dimension of the KV tensor must be contiguous")
    s = t.stride()
    if fmt == "vllm":
        L, _, T, H, D = t.shape
        return (L, T, H, D), (s[0], s[1], s[2], s[3])
    if fmt == "huggingface":
        L, _, H, T, D = t.shape
        return (L, T, H, D), (s[0], s[1], s[3], s[2])
    raise ValueError("Invalid KV format: %s" % fmt)


@dataclass
class EncodedKV:
    """Device-resident result of `encode_kv` (one flat payload for the whole tensor)."""
    cdf: torch.Tensor          # int16 [nchunks, 2L, C, Lp]
    maxima: torch.Tensor       # 16-bit [2, L, T]: row maxima of K and V
    lengths: torch.Tensor      # int32 [nsub, 2L, C]
    offsets: torch.Tensor      # int64 [nsub*2L*C + 1], exclusive running sum of lengths
    payload: torch.Tensor      # uint8 [>= total bytes]; streams back to back
    status: torch.Tensor       # int32 [1]; non-zero if a stream overflowed 256 bytes
    num_layers: int
    num_tokens: int
    num_heads: int
    head_size: int
    chunk_tokens: int
    max_bins: int
    delta_group: int = 0       # > 0: delta-against-anchor groups (not part of the reference codec)

    @property
    def num_chunks(self):
        return -(-self.num_tokens // self.chunk_tokens)

    @property
    def subchunks_per_chunk(self):
        return -(-self.chunk_tokens // MAX_TOKENS_PER_STREAM)

    def sub_boundaries(self):
        """Host list of payload offsets at every sub-chunk boundary (one device read)."""
        per_sub = 2 * self.num_layers * self.num_heads * self.head_size
        idx = torch.arange(0, self.lengths.shape[0] + 1, device=self.offsets.device) * per_sub
        return self.offsets[idx].tolist()

    def total_bytes(self):
        return int(self.offsets[-1].item())

    def check(self):
        self.raise_for_status(int(self.status.item()))

    @staticmethod
    def raise_for_status(st):
        """st: the status word as read back from the device."""
        if st & 1:
            raise RuntimeError("a stream exceeded %d bytes (the reference overruns its buffer there)"
                               % MAX_TOKENS_PER_STREAM)
        if st & 2:
            raise RuntimeError("payload buffer too small")

    def chunk(self, i, boundaries=None):
        """(cdf [2L,C,Lp], max_k [L,Tc,1], max_v [L,Tc,1], [(bytestream, lengths, ntokens)...])
        for chunk i: the fields of the reference's CacheGenGPUEncoderOutput."""
        if boundaries is None:
            boundaries = self.sub_boundaries()
        t0 = i * self.chunk_tokens
        t1 = min(t0 + self.chunk_tokens, self.num_tokens)
        g0 = i * self.subchunks_per_chunk
        subs = []
        for j, start in enumerate(range(t0, t1, MAX_TOKENS_PER_STREAM)):
            g = g0 + j
            subs.append((self.payload[boundaries[g]:boundaries[g + 1]], self.lengths[g],
                         min(MAX_TOKENS_PER_STREAM, t1 - start)))
        return (self.cdf[i], self.maxima[0, :, t0:t1, None], self.maxima[1, :, t0:t1, None], subs)


def num_subchunks(num_tokens, chunk_tokens):
    return int(_lib.lib().cg_num_subchunks(num_tokens, chunk_tokens))


def encode_workspace_bytes(num_layers, num_tokens, num_channels, chunk_tokens):
    return int(_lib.lib().cg_encode_kv_workspace(num_layers, num_tokens, num_channels, chunk_tokens))


def encode_kv(kv, key_bins, value_bins, chunk_tokens=None, fmt="vllm", max_bins=None,
              workspace=None, out: Optional[EncodedKV] = None, delta_group=0, _test_flags=None):
    """kv: fp16/bf16 GPU tensor [L,2,T,H,D] (fmt "vllm") or [L,2,H,T,D] ("huggingface").
    key_bins / value_bins: float32 GPU tensors [L].  chunk_tokens: tokens per table
    (default: all T, i.e. one `to_bytes` call).  `workspace` (uint8, GPU) and `out`
    (a previous result of the same geometry) let a caller reuse memory.  delta_group > 0
    switches on delta-against-anchor quantization in token groups of that size (an extension:
    the reference codec has none); decode with the same value.  `_test_flags` (tests only) goes to the
    library's test entry point, which takes the same arguments and must give the same results."""
    if not kv.is_cuda:
        raise RuntimeError("KV tensor should be on GPU")
    if kv.dtype not in _DT:
        raise RuntimeError("KV tensor must be float16 or bfloat16")
    (L, T, H, D), (sl, skv, st, sh) = _kv_strides(kv, fmt)
    if key_bins.numel() != L or value_bins.numel() != L:
        raise RuntimeError("bins vectors must have one entry per layer (%d)" % L)
    C = H * D
    S = int(chunk_tokens) if chunk_tokens else T
    if max_bins is None:
        max_bins = int(max(float(key_bins.max()), float(value_bins.max())))
    dev = kv.device
    lib = _lib.lib()
    nchunks = int(lib.cg_num_chunks(T, S))
    nsub = int(lib.cg_num_subchunks(T, S))
    nstreams = nsub * 2 * L * C
    key_bins = key_bins.to(device=dev, dtype=torch.float32).contiguous()
    value_bins = value_bins.to(device=dev, dtype=torch.float32).contiguous()
    ws_bytes = int(lib.cg_encode_kv_workspace(L, T, C, S))
    if workspace is None or workspace.numel() < ws_bytes:
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    if out is None:
        out = EncodedKV(
            cdf=torch.empty((nchunks, 2 * L, C, max_bins + 1), dtype=torch.int16, device=dev),
            maxima=torch.empty((2, L, T), dtype=kv.dtype, device=dev),
            lengths=torch.empty((nsub, 2 * L, C), dtype=torch.int32, device=dev),
            offsets=torch.empty(nstreams + 1, dtype=torch.int64, device=dev),
            payload=torch.empty(nstreams * MAX_TOKENS_PER_STREAM, dtype=torch.uint8, device=dev),
            status=torch.empty(1, dtype=torch.int32, device=dev),
            num_layers=L, num_tokens=T, num_heads=H, head_size=D, chunk_tokens=S, max_bins=max_bins,
            delta_group=int(delta_group))
    else:
        # a reused result must have been made for this geometry: the kernels write every field
        want = {"cdf": (nchunks, 2 * L, C, max_bins + 1), "maxima": (2, L, T), "lengths": (nsub, 2 * L, C),
                "offsets": (nstreams + 1,), "status": (1,)}
        for name, shape in want.items():
            t = getattr(out, name)
            if tuple(t.shape) != shape or not t.is_contiguous() or t.device != dev:
                raise RuntimeError("encode_kv: `out.%s` has shape %s, this call needs %s (contiguous, on %s)"
                                   % (name, tuple(t.shape), shape, dev))
        if out.maxima.dtype != kv.dtype or out.cdf.dtype != torch.int16 or out.lengths.dtype != torch.int32 \
                or out.offsets.dtype != torch.int64 or out.payload.dtype != torch.uint8 or out.status.dtype != torch.int32:
            raise RuntimeError("encode_kv: `out` holds tensors of the wrong dtype for this call")
        if not out.payload.is_contiguous() or out.payload.device != dev:
            raise RuntimeError("encode_kv: `out.payload` must be a contiguous tensor on %s" % dev)
        if (out.num_layers, out.num_tokens, out.num_heads, out.head_size, out.chunk_tokens, out.max_bins,
                out.delta_group) != (L, T, H, D, S, max_bins, int(delta_group)):
            raise RuntimeError("encode_kv: `out` was made for another geometry")
    with torch.cuda.device(dev):
        args = (kv.data_ptr(), _DT[kv.dtype], L, T, H, D, sl, skv, st, sh,
                key_bins.data_ptr(), value_bins.data_ptr(), max_bins, S, int(delta_group),
                out.cdf.data_ptr(), out.maxima.data_ptr(), out.lengths.data_ptr(), out.offsets.data_ptr(),
                out.payload.data_ptr(), out.payload.numel(), out.status.data_ptr(),
                workspace.data_ptr(), workspace.numel(), _stream())
        if _test_flags is None:
            _lib.check(lib.cg_encode_kv(*args))
        else:
            _lib.check(lib.cg_test_encode_kv(*args, int(_test_flags)))
    return out


def scan_lengths(lengths):
    """int32 lengths (any shape) -> int64 [n+1] exclusive running sum on the GPU."""
    flat = lengths.contiguous().view(-1)
    n = flat.numel()
    lib = _lib.lib()
    offsets = torch.empty(n + 1, dtype=torch.int64, device=flat.device)
    scratch = torch.empty(int(lib.cg_scan_workspace(n)), dtype=torch.uint8, device=flat.device)
    with torch.cuda.device(flat.device):
        _lib.check(lib.cg_scan_lengths(flat.data_ptr(), n, offsets.data_ptr(), scratch.data_ptr(),
                                       scratch.numel(), _stream()))
    return offsets


def decode_kv(cdf, maxima, offsets, payload, key_bins, value_bins, num_layers, num_tokens,
              num_heads, head_size, chunk_tokens, fmt="vllm", out_dtype=None, out=None, delta_group=0):
    """Inverse of `encode_kv`: returns the dequantized KV tensor, [L,2,T,H,D] for fmt "vllm"
    (default dtype bfloat16) or [L,2,H,T,D] for "huggingface" (default float16), as
    cachegen_decoder.py:169-173 does."""
    L, T, H, D = num_layers, num_tokens, num_heads, head_size
    dev = cdf.device
    if out_dtype is None:
        out_dtype = torch.bfloat16 if fmt == "vllm" else torch.float16
    if out is None:
        shape = (L, 2, T, H, D) if fmt == "vllm" else (L, 2, H, T, D)
        out = torch.empty(shape, dtype=out_dtype, device=dev)
    (L2, T2, H2, D2), (ol, okv, ot, oh) = _kv_strides(out, fmt)
    if (L2, T2, H2, D2) != (L, T, H, D) or out.dtype not in _DT:
        raise RuntimeError("output tensor does not match the encoded geometry")
    cdf = cdf.contiguous()
    maxima = maxima.contiguous()
    if maxima.dtype not in _DT:
        raise RuntimeError("row maxima must be float16 or bfloat16")
    # the kernel indexes every input by the geometry: refuse inputs that do not have it
    S = int(chunk_tokens)
    if S <= 0:
        raise RuntimeError("chunk_tokens must be positive")
    C = H * D
    nchunks, nsub = -(-T // S), num_subchunks(T, S)
    if key_bins.numel() != L or value_bins.numel() != L:
        raise RuntimeError("bins vectors must have one entry per layer (%d), got %d and %d"
                           % (L, key_bins.numel(), value_bins.numel()))
    if cdf.dim() != 4 or tuple(cdf.shape[:3]) != (nchunks, 2 * L, C) or cdf.dtype != torch.int16:
        raise RuntimeError("tables must be int16 [%d, %d, %d, Lp], got %s %s"
                           % (nchunks, 2 * L, C, cdf.dtype, tuple(cdf.shape)))
    if tuple(maxima.shape) != (2, L, T):
        raise RuntimeError("row maxima must have shape (2, %d, %d), got %s" % (L, T, tuple(maxima.shape)))
    if offsets.dtype != torch.int64 or offsets.numel() != nsub * 2 * L * C + 1 or not offsets.is_contiguous():
        raise RuntimeError("offsets must be a contiguous int64 tensor of %d entries, got %s of %d"
                           % (nsub * 2 * L * C + 1, offsets.dtype, offsets.numel()))
    if payload.dtype != torch.uint8 or not payload.is_contiguous() or payload.numel() == 0:
        raise RuntimeError("payload must be a contiguous, non-empty uint8 tensor")
    for name, t in (("maxima", maxima), ("offsets", offsets), ("payload", payload)):
        if t.device != dev:
            raise RuntimeError("%s is on %s, the tables on %s" % (name, t.device, dev))
    key_bins = key_bins.to(device=dev, dtype=torch.float32).contiguous()
    value_bins = value_bins.to(device=dev, dtype=torch.float32).contiguous()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().cg_decode_kv(
            cdf.data_ptr(), cdf.shape[-1] - 1, maxima.data_ptr(), _DT[maxima.dtype],
            offsets.data_ptr(), payload.data_ptr(), payload.numel(),
            key_bins.data_ptr(), value_bins.data_ptr(), L, T, H, D, int(chunk_tokens), int(delta_group),
            out.data_ptr(), _DT[out.dtype], ol, okv, ot, oh, _stream()))
    return out


def decode_encoded(enc: EncodedKV, key_bins, value_bins, fmt="vllm", out_dtype=None, out=None):
    return decode_kv(enc.cdf, enc.maxima, enc.offsets, enc.payload, key_bins, value_bins,
                     enc.num_layers, enc.num_tokens, enc.num_heads, enc.head_size,
                     enc.chunk_tokens, fmt=fmt, out_dtype=out_dtype, out=out, delta_group=enc.delta_group)


def quantize_kv(kv, key_bins, value_bins, fmt="vllm"):
    """torch_quant_vectorized on K and V (cachegen_encoder.py:42-59): returns
    (symbols uint8 [2L,T,C], maxima [2,L,T] in kv.dtype)."""
    (L, T, H, D), (sl, skv, st, sh) = _kv_strides(kv, fmt)
    dev = kv.device
    sym = torch.empty((2 * L, T, H * D), dtype=torch.uint8, device=dev)
    maxima = torch.empty((2, L, T), dtype=kv.dtype, device=dev)
    key_bins = key_bins.to(device=dev, dtype=torch.float32).contiguous()
    value_bins = value_bins.to(device=dev, dtype=torch.float32).contiguous()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().cg_quantize_kv(
            kv.data_ptr(), _DT[kv.dtype], L, T, H, D, sl, skv, st, sh,
            key_bins.data_ptr(), value_bins.data_ptr(), sym.data_ptr(), maxima.data_ptr(), _stream()))
    return sym, maxima


def encode_levels_workspace_bytes(num_layers, num_tokens, num_channels, chunk_tokens, num_levels):
    return int(_lib.lib().cg_encode_kv_levels_workspace(num_layers, num_tokens, num_channels, chunk_tokens, num_levels))


def encode_kv_levels(kv, levels, chunk_tokens=None, fmt="vllm", workspace=None, max_bins=None, out=None):
    """Encode the same KV cache at several quantization levels from one read of the tensor (the
    adaptive-streaming use of the reference: src/utils.py:357-377 and run_adaptation.py:63-72
    pre-encode every chunk at QUANT_LEVEL 1..3, one serializer call per level).  `levels` is a
    list of (key_bins, value_bins); `max_bins` an optional list of table sizes (default: each
    level's largest bins value).  Returns one EncodedKV per level; they share the row maxima
    (which do not depend on the level) and nothing else, and each equals what `encode_kv` gives
    for that level.  `out`: a previous result of the same call, to reuse its tensors."""
    import ctypes
    if not kv.is_cuda:
        raise RuntimeError("KV tensor should be on GPU")
    if kv.dtype not in _DT:
        raise RuntimeError("KV tensor must be float16 or bfloat16")
    (L, T, H, D), (sl, skv, st, sh) = _kv_strides(kv, fmt)
    C = H * D
    S = int(chunk_tokens) if chunk_tokens else T
    n = len(levels)
    lib = _lib.lib()
    if not 1 <= n <= 8:
        raise RuntimeError("between 1 and 8 levels, got %d" % n)
    dev = kv.device
    bins = []
    for kb, vb in levels:
        if kb.numel() != L or vb.numel() != L:
            raise RuntimeError("bins vectors must have one entry per layer (%d)" % L)
        bins.append((kb.to(device=dev, dtype=torch.float32).contiguous(), vb.to(device=dev, dtype=torch.float32).contiguous()))
    if max_bins is None:
        max_bins = [int(max(float(kb.max()), float(vb.max()))) for kb, vb in levels]
    if len(max_bins) != n:
        raise RuntimeError("max_bins must have one entry per level")
    nchunks = int(lib.cg_num_chunks(T, S))
    nsub = int(lib.cg_num_subchunks(T, S))
    nstreams = nsub * 2 * L * C
    ws_bytes = int(lib.cg_encode_kv_levels_workspace(L, T, C, S, n))
    if workspace is None or workspace.numel() < ws_bytes:
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    if out is None:
        maxima = torch.empty((2, L, T), dtype=kv.dtype, device=dev)
        status = torch.empty(n, dtype=torch.int32, device=dev)
        out = [EncodedKV(
            cdf=torch.empty((nchunks, 2 * L, C, mb + 1), dtype=torch.int16, device=dev),
            maxima=maxima,
            lengths=torch.empty((nsub, 2 * L, C), dtype=torch.int32, device=dev),
            offsets=torch.empty(nstreams + 1, dtype=torch.int64, device=dev),
            payload=torch.empty(nstreams * MAX_TOKENS_PER_STREAM, dtype=torch.uint8, device=dev),
            status=status[v:v + 1],
            num_layers=L, num_tokens=T, num_heads=H, head_size=D, chunk_tokens=S, max_bins=mb)
            for v, mb in enumerate(max_bins)]
    else:
        if len(out) != n:
            raise RuntimeError("encode_kv_levels: `out` holds %d levels, this call %d" % (len(out), n))
        for e, mb in zip(out, max_bins):
            if (e.num_layers, e.num_tokens, e.num_heads, e.head_size, e.chunk_tokens, e.max_bins) != (L, T, H, D, S, mb) \
                    or e.maxima.data_ptr() != out[0].maxima.data_ptr() or e.maxima.dtype != kv.dtype \
                    or tuple(e.cdf.shape) != (nchunks, 2 * L, C, mb + 1) or e.lengths.numel() != nstreams:
                raise RuntimeError("encode_kv_levels: `out` was made for another geometry")
        if any(out[v].status.data_ptr() != out[0].status.data_ptr() + 4 * v for v in range(n)):
            raise RuntimeError("encode_kv_levels: `out` must come from a previous encode_kv_levels call")

    def ptrs(ctype, values):
        return (ctype * n)(*values)

    with torch.cuda.device(dev):
        _lib.check(lib.cg_encode_kv_levels(
            kv.data_ptr(), _DT[kv.dtype], L, T, H, D, sl, skv, st, sh, n,
            ptrs(ctypes.c_void_p, [kb.data_ptr() for kb, _ in bins]), ptrs(ctypes.c_void_p, [vb.data_ptr() for _, vb in bins]),
            ptrs(ctypes.c_int, max_bins), S,
            ptrs(ctypes.c_void_p, [e.cdf.data_ptr() for e in out]), out[0].maxima.data_ptr(),
            ptrs(ctypes.c_void_p, [e.lengths.data_ptr() for e in out]),
            ptrs(ctypes.c_void_p, [e.offsets.data_ptr() for e in out]),
            ptrs(ctypes.c_void_p, [e.payload.data_ptr() for e in out]),
            ptrs(ctypes.c_int64, [e.payload.numel() for e in out]),
            out[0].status.data_ptr(), workspace.data_ptr(), workspace.numel(), _stream()))
    return out
