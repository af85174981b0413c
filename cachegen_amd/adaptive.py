"""Adaptive streaming of an encoded KV cache: per-chunk choice of the quantization level under a
time-to-first-token budget, and reassembly of the chosen chunks.

Mirrors the reference's streaming adaptation (src/utils.py:284-377, run_adaptation.py:63-116):
every chunk of the context is encoded at the three quantization levels of the 7B table; for each
chunk the controller takes the best level whose transfer time at the chunk's bandwidth fits an
equal share of the SLO, or falls back to recomputing the chunk (level 0) at a fixed delay.  The
reference reads the encoded chunks back from one pickle file per (document, chunk, level); here
the same decisions are made on the sizes of in-memory blobs, all levels are encoded in one pass
over the cache (`codec.encode_kv_levels`), and the chosen chunks are decoded straight into their
token range of one output tensor instead of being concatenated layer by layer.
"""
import os
import random
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

QUANT_LEVELS = (1, 2, 3)            # cachegen_basics.py:33-69; 3 is the finest


def bw_generator(num_chunks: int, rng: Optional[random.Random] = None) -> np.ndarray:
    """One bandwidth (Gbps) per chunk, uniform in [0.1, 10] (src/utils.py:284-292)."""
    rng = rng or random
    return np.array([rng.uniform(0.1, 10) for _ in range(num_chunks)])


def config_selection(all_bws: Sequence[float], chunk_delay: float, slo: float, chunk_size: int, length: int,
                     blob_sizes: Sequence[Dict[int, int]]) -> Tuple[float, List[int]]:
    """src/utils.py:294-317 with the pickle files replaced by their sizes.

    all_bws[i]: bandwidth in Gbps while chunk i is sent; blob_sizes[i][level]: bytes of chunk i
    encoded at `level`.  Returns (time to first token in seconds, level per chunk); level 0 means
    the chunk is recomputed, which costs `chunk_delay` seconds.  A chunk's budget is slo /
    round(length / chunk_size) and must be met strictly, levels are tried from 3 down to 1, and a
    context that is not a whole number of chunks has its tail chunk considered too, all as in the
    reference."""
    num_chunks = round(length / chunk_size)
    ttft = 0.0
    configs: List[int] = []
    for chunk_id, _ in enumerate(range(0, length, chunk_size)):
        bw = all_bws[chunk_id]
        found = False
        for level in (3, 2, 1):
            seconds = blob_sizes[chunk_id][level] / 1e9 * 8 / bw
            if seconds < slo / num_chunks:
                ttft += seconds
                configs.append(level)
                found = True
                break
        if not found:
            ttft += chunk_delay
            configs.append(0)
    return ttft, configs


def level_bins(level: int, model_name: str = "mistralai/Mistral-7B-Instruct-v0.2"):
    """(key_bins, value_bins) float32 [L] of one QUANT_LEVEL of the 7B table, without touching
    the process environment for the caller (cachegen_basics.py:27-69 reads QUANT_LEVEL)."""
    from .serde import cachegen_basics as basics
    saved = os.environ.get("QUANT_LEVEL")
    os.environ["QUANT_LEVEL"] = str(level)
    try:
        config = basics.CacheGenConfig.from_model_name(model_name)
    finally:
        if saved is None:
            del os.environ["QUANT_LEVEL"]
        else:
            os.environ["QUANT_LEVEL"] = saved
    if config is None:
        raise ValueError(f"Invalid quantization level: {level}")
    return basics.make_key_bins(config), basics.make_value_bins(config)


def encode_levels(kv: torch.Tensor, chunk_size: int, levels: Sequence[int] = QUANT_LEVELS, fmt: str = "vllm",
                  model_name: str = "mistralai/Mistral-7B-Instruct-v0.2", compact: bool = True) -> List[Dict[int, bytes]]:
    """What the encode half of run_adaptation.py:63-72 leaves on disk, kept in memory:
    blobs[chunk][level] = the chunk's flat wire container at that level (version 2 unless
    compact=False).  The cache is read once per level for all of its chunks."""
    from . import codec
    from .serde import wire
    tables = [level_bins(level, model_name) for level in levels]
    encoded = codec.encode_kv_levels(kv, tables, chunk_tokens=chunk_size, fmt=fmt)
    blobs: List[Dict[int, bytes]] = [dict() for _ in range(encoded[0].num_chunks)]
    for level, enc in zip(levels, encoded):
        for i, blob in enumerate(wire.pack_chunks(enc, compact=compact)):
            blobs[i][level] = blob
    return blobs


def merge(configs: Sequence[int], blobs: Sequence[Dict[int, bytes]], chunk_size: int, length: int,
          orig_kv: Optional[torch.Tensor] = None, fmt: str = "vllm", out_dtype=None,
          model_name: str = "mistralai/Mistral-7B-Instruct-v0.2") -> torch.Tensor:
    """src/utils.py:360-377: the KV cache rebuilt from the chosen level of every whole chunk
    (a partial tail chunk is dropped, as there); level 0 takes the chunk from `orig_kv`.
    Returns one tensor [L, 2, T', H, D] (fmt "vllm") or [L, 2, H, T', D] ("huggingface") with
    T' = chunk_size * (length // chunk_size), in `out_dtype` (default: the dtype of `orig_kv`, else
    bfloat16 for "vllm" and float16 for "huggingface" as the deserializer gives); every chunk is
    decoded in place into its token range."""
    from . import codec
    from .serde import wire
    nwhole = length // chunk_size
    if nwhole == 0:
        raise ValueError("context shorter than one chunk")
    out = None
    tdim = 2 if fmt == "vllm" else 3
    bins_cache = {}
    for chunk_id in range(nwhole):
        level = configs[chunk_id]
        t0, t1 = chunk_id * chunk_size, (chunk_id + 1) * chunk_size
        if level == 0:
            if orig_kv is None:
                raise ValueError(f"chunk {chunk_id} is to be recomputed but no original cache was given")
            piece = orig_kv.narrow(tdim, t0, chunk_size)
            if out is None:
                shape = list(orig_kv.shape)
                shape[tdim] = nwhole * chunk_size
                out = torch.empty(shape, dtype=out_dtype or orig_kv.dtype, device=orig_kv.device)
            out.narrow(tdim, t0, chunk_size).copy_(piece)
            continue
        blob = blobs[chunk_id][level]
        dev = orig_kv.device if orig_kv is not None and orig_kv.is_cuda else torch.device("cuda")
        h, cdf, maxima, lengths, payload = wire.unpack_to_device(blob, dev)
        if h["num_tokens"] != chunk_size:
            raise ValueError(f"chunk {chunk_id} holds {h['num_tokens']} tokens, expected {chunk_size}")
        if out is None:
            L, H, D = h["num_layers"], h["num_heads"], h["head_size"]
            shape = (L, 2, nwhole * chunk_size, H, D) if fmt == "vllm" else (L, 2, H, nwhole * chunk_size, D)
            dtype = out_dtype or (orig_kv.dtype if orig_kv is not None
                                  else (torch.bfloat16 if fmt == "vllm" else torch.float16))
            out = torch.empty(shape, dtype=dtype, device=dev)
        if level not in bins_cache:
            bins_cache[level] = level_bins(level, model_name)
        kb, vb = bins_cache[level]
        codec.decode_kv(cdf, maxima, codec.scan_lengths(lengths), payload, kb, vb, h["num_layers"],
                        chunk_size, h["num_heads"], h["head_size"], h["chunk_tokens"], fmt=fmt,
                        out=out.narrow(tdim, t0, chunk_size), delta_group=h["delta_group"])
    return out


def tensor_to_tuple(kv: torch.Tensor, layer_to_device_id: Optional[Dict[int, int]] = None):
    """[L, 2, H, T, D] -> tuple over layers of (key, value), each [1, H, T, D]
    (src/utils.py:167-175); with a device map every layer is moved to its device."""
    out = []
    for i in range(len(kv)):
        k, v = kv[i][0].unsqueeze(0), kv[i][1].unsqueeze(0)
        if layer_to_device_id is not None:
            k, v = k.to(f"cuda:{layer_to_device_id[i]}"), v.to(f"cuda:{layer_to_device_id[i]}")
        out.append((k, v))
    return tuple(out)


def to_blob(kv_tuples, device="cuda:0") -> torch.Tensor:
    """tuple over layers of (key, value) -> one tensor [L, 2, ...] (src/utils.py:118-121)."""
    return torch.stack([torch.stack(tuple(pair), dim=0).to(device) for pair in kv_tuples], dim=0)
