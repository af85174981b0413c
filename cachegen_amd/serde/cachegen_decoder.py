"""CacheGenDeserializer on MI355X
(LMCache/lmcache/storage_backend/serde/cachegen_decoder.py in the reference)."""
from typing import List

import torch

from .. import codec, torchac_hip
from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from . import cachegen_basics as CGBasics
from . import wire
from .cachegen_basics import CacheGenConfig, CacheGenGPUBytestream, CacheGenGPUEncoderOutput
from .serde import Deserializer


def decode_chunk(cdf: torch.Tensor, data_chunk: CacheGenGPUBytestream, target_buffer: torch.Tensor):
    """cachegen_decoder.py:52-75: decode one sub-chunk's streams into
    target_buffer [2L, ntokens, nchannels] (a strided view is fine)."""
    prefsum = codec.scan_lengths(data_chunk.bytestream_lengths)[1:].view(data_chunk.bytestream_lengths.shape)
    torchac_hip.decode_fast_prefsum(cdf, data_chunk.bytestream, prefsum, target_buffer)


def decode_function_gpu(cdf: torch.Tensor, data_chunks: List[CacheGenGPUBytestream],
                        layers_in_key: int, chunk_size: int, output: torch.Tensor):
    """cachegen_decoder.py:77-112: symbols of every sub-chunk -> (key, value) float32
    [layers_in_key, chunk_size, nchannels]."""
    nlayers, nchannels, _ = cdf.shape
    output = output.reshape((nlayers, chunk_size, nchannels))
    start = 0
    for data_chunk in data_chunks:
        end = start + data_chunk.ntokens
        decode_chunk(cdf, data_chunk, output[:, start:end, :])
        start = end
    out = output.reshape((2, layers_in_key, chunk_size, nchannels))
    key, value = out.float()
    return key, value


def do_dequantize(t: torch.Tensor, bins: torch.Tensor, maxtensors: torch.Tensor):
    """cachegen_decoder.py:24-34 (plain tensor ops; the fused path does this in-kernel)."""
    C = (bins // 2 - 1)[:, None, None]
    t = t - C
    t = t / C
    t = t * maxtensors
    return t


class CacheGenDeserializer(Deserializer):
    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata):
        self.cachegen_config = CacheGenConfig.from_model_name(metadata.model_name)
        self.chunk_size = config.chunk_size
        self.fmt = metadata.fmt
        self.key_bins = self.make_key_bins(self.cachegen_config)
        self.value_bins = self.make_value_bins(self.cachegen_config)

    def make_key_bins(self, config: CacheGenConfig) -> torch.Tensor:
        return CGBasics.make_key_bins(config).cuda()

    def make_value_bins(self, config: CacheGenConfig) -> torch.Tensor:
        return CGBasics.make_value_bins(config).cuda()

    def from_bytes(self, bs: bytes) -> torch.Tensor:
        """Returns bfloat16 [num_layers, 2, num_tokens, num_heads, head_size] for fmt "vllm",
        float16 [num_layers, 2, num_heads, num_tokens, head_size] for "huggingface"
        (cachegen_decoder.py:144-173).  Decode, dequantization, cast and layout are one
        kernel.  Blobs in the flat container of `wire` are recognised by their magic."""
        return self._decode(bs, None)

    def from_bytes_into(self, bs: bytes, out: torch.Tensor) -> torch.Tensor:
        """Decodes `bs` straight into `out`: a tensor, or a view into a larger one, of the
        chunk's shape in this deserializer's layout, float16 or bfloat16 (not in the reference,
        whose callers concatenate the decoded chunks)."""
        return self._decode(bs, out)

    def chunk_shape(self, bs: bytes):
        """Shape `from_bytes(bs)` would have, read from a flat container's header without
        decoding; None for a pickle container."""
        if not wire.is_flat(bs):
            return None
        h = wire.read_header(bs)
        L, T, H, D = h["num_layers"], h["num_tokens"], h["num_heads"], h["head_size"]
        return (L, 2, T, H, D) if self.fmt == "vllm" else (L, 2, H, T, D)

    def _decode(self, bs, out):
        if wire.is_flat(bs):
            return self._from_flat(bs, out)
        encoder_output = CacheGenGPUEncoderOutput.from_bytes(bs)
        cdf = encoder_output.cdf.cuda()
        max_k = encoder_output.max_tensors_key.cuda()
        max_v = encoder_output.max_tensors_value.cuda()
        nlayers, ntokens = max_k.shape[0], max_k.shape[1]
        chunks = encoder_output.data_chunks
        if len(chunks) == 1:
            payload = chunks[0].bytestream.cuda()
            lengths = chunks[0].bytestream_lengths.cuda()
        else:
            payload = torch.cat([c.bytestream.cuda() for c in chunks])
            lengths = torch.stack([c.bytestream_lengths.cuda() for c in chunks])
        offsets = codec.scan_lengths(lengths)
        maxima = torch.stack([max_k.reshape(nlayers, ntokens), max_v.reshape(nlayers, ntokens)])
        return codec.decode_kv(cdf.unsqueeze(0), maxima, offsets, payload, self.key_bins,
                               self.value_bins, nlayers, ntokens, encoder_output.num_heads,
                               encoder_output.head_size, chunk_tokens=ntokens, fmt=self.fmt, out=out)

    def _from_flat(self, bs, out=None) -> torch.Tensor:
        # the container's own consistency (stream lengths against the payload size) is checked on
        # the host inside unpack_to_device; the decode is queued before anything waits for the device
        h, cdf, maxima, lengths, payload = wire.unpack_to_device(bs, self.key_bins.device, defer_checks=True)
        if h["num_layers"] != self.key_bins.numel():
            raise ValueError("blob has %d layers, this deserializer's model %d"
                             % (h["num_layers"], self.key_bins.numel()))
        # a stream occupies min(length, 256) bytes of the payload (wire.py checks the same sum)
        offsets = codec.scan_lengths(lengths.clamp(max=wire.MAX_STREAM_BYTES))
        result = codec.decode_kv(cdf, maxima, offsets, payload, self.key_bins, self.value_bins,
                                 h["num_layers"], h["num_tokens"], h["num_heads"], h["head_size"],
                                 chunk_tokens=h["chunk_tokens"], fmt=self.fmt, delta_group=h["delta_group"],
                                 out=out)
        h["check"]()
        return result
