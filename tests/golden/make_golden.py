"""Writes tests/golden/*.json and *.npz.

Two kinds of vectors, kept apart on purpose:

* known_answers.json -- inputs and expected outputs derived BY HAND from the algorithm as
  written in the reference sources (LMCache/third_party/torchac_cuda/torchac_kernel_enc_new.cu
  :255-307, torchac_kernel_dec_new.cu:259-302, cal_cdf.cu:11-49, and
  LMCache/lmcache/storage_backend/serde/cachegen_encoder.py:54-57, cachegen_decoder.py:30-34).
  The reference itself holds no golden vectors for the codec and cannot run in this image
  (CUDA extension, no GPU toolchain for it), so none of these were produced by running it.
  This script only stores them; it does not compute them.

* regression_kv.npz -- a small seeded KV cache pushed through the CPU oracle
  (oracle/cachegen_oracle.c).  It is a regression fixture for the oracle and a second,
  file-based reference for the HIP path; it pins nothing the oracle's own pins do not.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

KNOWN_ANSWERS = {
    "quantize": [
        # MAX = bins//2 - 1; factor = MAX / max|row|; symbol = round_half_even(x*factor + MAX)
        {"bins": 32, "row": [1.0, -1.0, 0.5, 0.0], "symbols": [30, 0, 22, 15], "max": 1.0},
        {"bins": 16, "row": [1.0, -1.0, 0.5, 0.0], "symbols": [14, 0, 10, 7], "max": 1.0},
        {"bins": 12, "row": [1.0, -1.0, 0.5, 0.0], "symbols": [10, 0, 8, 5], "max": 1.0},
        {"bins": 32, "row": [0.0, 0.0, 0.0, 0.0], "symbols": [0, 0, 0, 0], "max": 0.0},
    ],
    "cdf": [
        # cum = [0,2,3,...,3,4,4]; cdf[i] = floor(65503*cum[i]/4) + i
        {"max_bins": 32, "symbols": [0, 0, 1, 30],
         "cdf": [0, 32752] + [49127 + i for i in range(2, 31)] + [65534, 65535]},
    ],
    "coder": [
        # cdf, symbols, expected bytes; bit strings in the comments are what the loop emits
        {"cdf": [0, 32768, 65535], "symbols": [0], "bytes": [0x20]},          # 0 | 01
        {"cdf": [0, 32768, 65535], "symbols": [1], "bytes": [0xA0]},          # 1 | 01
        {"cdf": [0, 32768, 65535], "symbols": [], "bytes": [0x40]},           # 01
        {"cdf": [0, 16384, 49152, 65535], "symbols": [1, 0], "bytes": [0x48]},   # pending, 01 0 | 01
        {"cdf": [0, 16384, 49152, 65535], "symbols": [1, 2], "bytes": [0xA8]},   # pending, 10 1 | 01
        {"cdf": [0, 16384, 49152, 65535], "symbols": [1] * 40,
         "bytes": list(int("0" + "1" * 41 + "000000", 2).to_bytes(6, "big"))},    # 40 pending: 0 then 41 ones
        # a table that is not dyadic, so that span * c is not a multiple of 2^16 and the floor of
        # `(span * c) >> 16` matters (worked through step by step in tests/test_oracle_pins.py:
        # rounding to nearest instead of truncating gives the five bytes 00 07 00 30 ff)
        {"cdf": [0, 7, 65535], "symbols": [1, 0, 1, 0, 0], "bytes": [0x00, 0x07, 0x00, 0x30, 0xFF, 0x00]},
    ],
    "decoder_boundary": [
        # hand-built streams (not encoder output) whose code value sits exactly on, and one below,
        # a symbol boundary low + floor(span * c / 2^16) with a dropped fraction above one half:
        # 12 zero bits, then the 32-bit value, zero fill
        {"cdf": [0, 7, 65535], "bytes": [0x00, 0x07, 0x00, 0x30, 0xFE, 0xA0], "symbols": [1, 0, 1]},   # value 0x70030FEA
        {"cdf": [0, 7, 65535], "bytes": [0x00, 0x07, 0x00, 0x30, 0xFE, 0x90], "symbols": [1, 0, 0]},   # value 0x70030FE9
    ],
    "dequantize": [
        # ((s - C) / C) * max in float32, then nearest-even to float16; C = bins//2 - 1
        {"bins": 32, "max": 1.0, "symbols": [22, 0, 30, 15],
         "float16_bits": [int(np.float16(np.float32(7) / np.float32(15)).view(np.uint16)), 0xBC00, 0x3C00, 0x0000]},
    ],
}


def main():
    with open(os.path.join(HERE, "known_answers.json"), "w") as f:
        json.dump(KNOWN_ANSWERS, f, indent=1)

    import torch
    from cachegen_amd.kvgen import make_kv
    from oracle import cachegen_oracle as oracle
    L, T, H, D = 2, 300, 2, 32
    kv = make_kv(L, T, H, D, seed=77)
    bits = kv.reshape(L, 2, T, H * D).view(torch.int16).numpy().view(np.uint16)
    kb = np.array([32.0, 16.0], dtype=np.float32)
    vb = np.array([12.0, 32.0], dtype=np.float32)
    enc = oracle.encode_function(bits, kb, vb)
    _, out = oracle.decode_function(enc, kb, vb, out_dt=oracle.DT_F16)
    np.savez_compressed(
        os.path.join(HERE, "regression_kv.npz"),
        kv_bits=bits, key_bins=kb, value_bins=vb, cdf=enc["cdf"],
        max_key=enc["max_tensors_key"], max_value=enc["max_tensors_value"],
        lengths=np.stack([c[1] for c in enc["data_chunks"]]),
        payload=np.concatenate([c[0] for c in enc["data_chunks"]]),
        ntokens=np.array([c[2] for c in enc["data_chunks"]]),
        dequantized_f16_bits=out)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
