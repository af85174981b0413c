"""The four entry points of the reference's `torchac_cuda` extension, on MI355X.

Same names, argument order, dtypes, shapes and in-place behaviour as the module
defined in LMCache/third_party/torchac_cuda/main.cpp:11-18; tensors must live on
the GPU, strides are honoured (the reference passes strided views:
cachegen_encoder.py:284, cachegen_decoder.py:106).  Work is queued on the current
torch stream.  Errors are RuntimeError, as TORCH_CHECK raises.
"""
import torch

from . import _lib

MAX_TOKENS_PER_STREAM = 256
MAX_BINS_SUPPORTED = 128


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def calculate_cdf(input, max_bins):
    """cal_cdf.cu:68-129. input int8/uint8 [nlayers, ntokens, nchannels] ->
    int16 [nlayers, nchannels, max_bins + 1]."""
    _require(input.is_cuda, "Input must be a CUDA tensor")
    _require(max_bins < MAX_BINS_SUPPORTED, "Max bins must be less than %d" % MAX_BINS_SUPPORTED)
    _require(input.dim() == 3 and input.dtype in (torch.int8, torch.uint8),
             "Input must be an int8 tensor of shape [nlayers, ntokens, nchannels]")
    nl, nt, nc = input.shape
    out = torch.zeros((nl, nc, max_bins + 1), dtype=torch.int16, device=input.device)
    if nl == 0 or nt == 0 or nc == 0:
        return out
    s = input.stride()
    with torch.cuda.device(input.device):
        _lib.check(_lib.lib().cg_calculate_cdf(input.data_ptr(), nl, nt, nc, s[0], s[1], s[2],
                                               int(max_bins), out.data_ptr(), _stream()))
    return out


def encode_fast_new(cdf, input_sym, output_buffer, output_lengths):
    """enc_new.cu:355-451. cdf int16 [nl, nc, Lp]; input_sym int8 [nl, ntokens<=256, nc];
    output_buffer uint8 [nl, nc, cap] and output_lengths int32 [nl, nc] are written."""
    _require(cdf.is_cuda, "CDF should be on GPU")
    _require(input_sym.is_cuda, "Input symbols should be on GPU")
    _require(output_buffer.is_cuda, "Output buffer should be on GPU")
    _require(output_lengths.is_cuda, "Output lengths should be on GPU")
    _require(cdf.dtype == torch.int16 and input_sym.dtype in (torch.int8, torch.uint8) and
             output_buffer.dtype == torch.uint8 and output_lengths.dtype == torch.int32,
             "expected cdf int16, symbols int8, output uint8, lengths int32")
    _require(cdf.shape[0] == input_sym.shape[0], "CDF and input should have the same number of layers")
    _require(cdf.shape[1] == input_sym.shape[2], "CDF and input should have the same number of channels")
    _require(output_buffer.shape[0] == cdf.shape[0], "Output buffer should have the same number of layers as CDF")
    _require(output_buffer.shape[1] == cdf.shape[1], "Output buffer should have the same number of channels as CDF")
    _require(output_lengths.shape[0] == cdf.shape[0], "Output lengths should have the same number of layers as CDF")
    _require(output_lengths.shape[1] == cdf.shape[1], "Output lengths should have the same number of channels as CDF")
    nl, nt, nc = input_sym.shape
    _require(nt <= MAX_TOKENS_PER_STREAM,
             "Number of tokens should be less than or equal to %d" % MAX_TOKENS_PER_STREAM)
    _require(output_buffer.stride(2) == 1 and output_lengths.is_contiguous(),
             "Output buffer rows and output lengths should be contiguous")
    cdf = cdf.contiguous()
    s = input_sym.stride()
    o = output_buffer.stride()
    with torch.cuda.device(cdf.device):
        _lib.check(_lib.lib().cg_encode_fast_new(
            cdf.data_ptr(), cdf.shape[2], input_sym.data_ptr(), nl, nt, nc, s[0], s[1], s[2],
            output_buffer.data_ptr(), output_buffer.shape[2], o[0], o[1],
            output_lengths.data_ptr(), _stream()))


def _check_decode(cdf, lengths, output):
    _require(cdf.is_cuda, "CDF should be on GPU")
    _require(lengths.is_cuda, "Lengths should be on GPU")
    _require(output.is_cuda, "Output should be on GPU")
    _require(cdf.shape[0] == lengths.shape[0], "CDF and lengths should have the same number of layers")
    _require(cdf.shape[1] == lengths.shape[1], "CDF and lengths should have the same number of channels")
    _require(cdf.shape[0] == output.shape[0], "CDF and output should have the same number of layers")
    _require(cdf.shape[1] == output.shape[2], "CDF and output should have the same number of channels")
    _require(output.shape[1] <= MAX_TOKENS_PER_STREAM,
             "Number of tokens should be less than or equal to %d" % MAX_TOKENS_PER_STREAM)
    _require(cdf.dtype == torch.int16 and output.dtype == torch.uint8, "expected cdf int16, output uint8")


def decode_fast_new(cdf, bytestreams, lengths, output):
    """dec_new.cu:314-393. bytestreams uint8 [nl, nc, cap] padded; lengths int32 [nl, nc];
    output uint8 [nl, ntokens, nc] is written."""
    _require(bytestreams.is_cuda, "Bytestreams should be on GPU")
    _check_decode(cdf, lengths, output)
    _require(bytestreams.dtype == torch.uint8 and lengths.dtype == torch.int32,
             "expected bytestreams uint8, lengths int32")
    _require(bytestreams.shape[0] == cdf.shape[0], "CDF and bytestreams should have the same number of layers")
    _require(bytestreams.shape[1] == cdf.shape[1], "CDF and bytestreams should have the same number of channels")
    _require(bytestreams.stride(2) == 1, "Bytestream rows should be contiguous")
    cdf = cdf.contiguous()
    lengths = lengths.contiguous()
    nl, nt, nc = output.shape
    if nt == 0:
        return
    p = bytestreams.stride()
    o = output.stride()
    with torch.cuda.device(cdf.device):
        _lib.check(_lib.lib().cg_decode_fast_new(
            cdf.data_ptr(), cdf.shape[2], bytestreams.data_ptr(), bytestreams.shape[2], p[0], p[1],
            lengths.data_ptr(), nl, nt, nc, output.data_ptr(), o[0], o[1], o[2], _stream()))


def decode_fast_prefsum(cdf, bytestreams, lengths_prefsum, output):
    """dec_new.cu:403-479. bytestreams uint8 [n] (streams back to back in (layer, channel)
    order); lengths_prefsum int64 [nl, nc], the inclusive running sum of the stream lengths;
    output uint8 [nl, ntokens, nc] is written."""
    _require(bytestreams.is_cuda, "Bytestreams should be on GPU")
    _check_decode(cdf, lengths_prefsum, output)
    _require(bytestreams.dtype == torch.uint8 and bytestreams.dim() == 1, "expected a 1-D uint8 bytestream")
    _require(lengths_prefsum.dtype == torch.int64, "expected int64 prefix sums")
    cdf = cdf.contiguous()
    bytestreams = bytestreams.contiguous()
    lengths_prefsum = lengths_prefsum.contiguous()
    nl, nt, nc = output.shape
    if nt == 0:
        return
    o = output.stride()
    with torch.cuda.device(cdf.device):
        _lib.check(_lib.lib().cg_decode_fast_prefsum(
            cdf.data_ptr(), cdf.shape[2], bytestreams.data_ptr(), bytestreams.numel(),
            lengths_prefsum.data_ptr(), nl, nt, nc, output.data_ptr(), o[0], o[1], o[2], _stream()))
