"""CacheGenSerializer on MI355X
(LMCache/lmcache/storage_backend/serde/cachegen_encoder.py in the reference)."""
import torch

from .. import codec, torchac_hip
from ..config import LMCacheEngineConfig, LMCacheEngineMetadata
from . import cachegen_basics as CGBasics
from . import wire
from .cachegen_basics import CacheGenConfig, CacheGenGPUBytestream, CacheGenGPUEncoderOutput
from .serde import Serializer


def torch_quant_vectorized(bins: torch.Tensor, input_groups: torch.Tensor):
    """cachegen_encoder.py:42-59 for one of K / V: bins float32 [nlayers], input_groups
    [nlayers, ntokens, nchannels] -> (int8 symbols, maxima [nlayers, ntokens, 1])."""
    nl, nt, nc = input_groups.shape
    kv = torch.stack([input_groups, input_groups], dim=1).view(nl, 2, nt, 1, nc)
    sym, maxima = codec.quantize_kv(kv, bins, bins, fmt="vllm")
    return sym[:nl].view(torch.int8), maxima[0].unsqueeze(-1)


def collect_bytes(output_buffer: torch.Tensor, output_lengths: torch.Tensor) -> torch.Tensor:
    """cachegen_encoder.py:209-222: the streams of a padded buffer, back to back."""
    cap = output_buffer.shape[-1]
    offsets = codec.scan_lengths(output_lengths)
    idx = torch.arange(int(offsets[-1].item()), device=output_buffer.device)
    stream = torch.searchsorted(offsets[1:], idx, right=True)
    return output_buffer.reshape(-1, cap)[stream, idx - offsets[stream]]


def encode_ntokens(cdf_int, encode_input, output_buffer, output_lengths) -> torch.Tensor:
    """cachegen_encoder.py:224-243."""
    torchac_hip.encode_fast_new(cdf_int, encode_input, output_buffer, output_lengths)
    return collect_bytes(output_buffer, output_lengths)


def encode_function(kv: torch.Tensor, config: CacheGenConfig, key_bins: torch.Tensor,
                    value_bins: torch.Tensor, chunk_size: int) -> CacheGenGPUEncoderOutput:
    """cachegen_encoder.py:247-301 for kv [num_layers, 2, num_tokens, num_heads, head_size]
    (any strides with a contiguous head): one table per (layer, channel) over all
    `chunk_size` tokens, one stream per (layer, channel, 256-token sub-chunk)."""
    num_heads, head_size = kv.shape[-2:]
    enc = codec.encode_kv(kv, key_bins, value_bins, chunk_tokens=chunk_size, fmt="vllm")
    enc.check()
    return _chunk_output(enc, 0, enc.sub_boundaries(), num_heads, head_size)


def _chunk_output(enc, i, bounds, num_heads, head_size) -> CacheGenGPUEncoderOutput:
    """Chunk i of an encoded tensor as the reference's container.  Every field is a tensor of
    its own: pickling a view would write out the whole buffer it is a view of."""
    cdf, max_k, max_v, subs = enc.chunk(i, bounds)
    data_chunks = [CacheGenGPUBytestream(bytestream=b.clone(), bytestream_lengths=l.clone(), ntokens=n)
                   for b, l, n in subs]
    return CacheGenGPUEncoderOutput(data_chunks, cdf.clone(), max_tensors_key=max_k.clone(),
                                    max_tensors_value=max_v.clone(), num_heads=num_heads, head_size=head_size)


class CacheGenSerializer(Serializer):
    def __init__(self, config: LMCacheEngineConfig, metadata: LMCacheEngineMetadata,
                 wire_format: str = "pickle"):
        """wire_format "pickle": the reference's container (cachegen_basics.py:110-122);
        "flat": the versioned flat container of `wire`; "compact": its version 2, which stores
        the tables of chunks of up to 256 tokens as histogram counts.  `CacheGenDeserializer`
        reads all three."""
        if wire_format not in ("pickle", "flat", "compact"):
            raise ValueError(f"Invalid wire format: {wire_format}")
        self.wire_format = wire_format
        self.cachegen_config = CacheGenConfig.from_model_name(metadata.model_name)
        self.chunk_size = config.chunk_size
        self.fmt = metadata.fmt
        self.key_bins = self.make_key_bins(self.cachegen_config)
        self.value_bins = self.make_value_bins(self.cachegen_config)

    def make_key_bins(self, config: CacheGenConfig) -> torch.Tensor:
        return CGBasics.make_key_bins(config).cuda()

    def make_value_bins(self, config: CacheGenConfig) -> torch.Tensor:
        return CGBasics.make_value_bins(config).cuda()

    def to_bytes(self, tensor: torch.Tensor) -> bytes:
        """tensor: [num_layers, 2, num_tokens, num_heads, head_size] for fmt "vllm",
        [num_layers, 2, num_heads, num_tokens, head_size] for "huggingface"; any device.
        The huggingface layout is read in place through strides (no permuted copy)."""
        if self.fmt == "huggingface":
            tensor = tensor.permute(0, 1, 3, 2, 4)
        ntokens = tensor.shape[2]
        if self.wire_format != "pickle":
            enc = codec.encode_kv(tensor.cuda(), self.key_bins, self.value_bins, chunk_tokens=ntokens)
            return wire.pack_chunks(enc, per_chunk=False, compact=self.wire_format == "compact")[0]
        output = encode_function(tensor.cuda(), self.cachegen_config, self.key_bins,
                                 self.value_bins, ntokens)
        return output.to_bytes()

    def to_bytes_chunks(self, tensor: torch.Tensor, chunk_size: int):
        """One blob per `chunk_size` tokens of `tensor` (same layouts as `to_bytes`), each equal
        to what `to_bytes` returns for that slice; all chunks are encoded in one pass over the
        tensor (not in the reference, whose callers loop over `to_bytes`)."""
        if self.fmt == "huggingface":
            tensor = tensor.permute(0, 1, 3, 2, 4)
        num_heads, head_size = tensor.shape[-2:]
        enc = codec.encode_kv(tensor.cuda(), self.key_bins, self.value_bins, chunk_tokens=chunk_size)
        if self.wire_format != "pickle":
            return wire.pack_chunks(enc, compact=self.wire_format == "compact")
        enc.check()
        bounds = enc.sub_boundaries()
        return [_chunk_output(enc, i, bounds, num_heads, head_size).to_bytes() for i in range(enc.num_chunks)]
