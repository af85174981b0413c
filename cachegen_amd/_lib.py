"""ctypes binding of lib/libcachegen_hip.so (declared in include/cachegen_hip.h).

There is no CPU or PyTorch fallback: if the library is missing, or a call fails,
a RuntimeError is raised.
"""
import ctypes
import os

from .build import LIBRARY

CG_OK = 0
DT_F16 = 0
DT_BF16 = 1

_c = ctypes
_P = _c.c_void_p
_I64 = _c.c_int64
_INT = _c.c_int
_SZ = _c.c_size_t

# name -> (restype, argtypes); mirrors include/cachegen_hip.h
SIGNATURES = {
    "cg_last_error": (_c.c_char_p, []),
    "cg_abi_version": (_INT, []),
    "cg_num_chunks": (_I64, [_I64, _I64]),
    "cg_num_subchunks": (_I64, [_I64, _I64]),
    "cg_calculate_cdf": (_INT, [_P, _I64, _I64, _I64, _I64, _I64, _I64, _INT, _P, _P]),
    "cg_encode_fast_new": (_INT, [_P, _INT, _P, _I64, _I64, _I64, _I64, _I64, _I64, _P, _I64, _I64, _I64, _P, _P]),
    "cg_decode_fast_new": (_INT, [_P, _INT, _P, _I64, _I64, _I64, _P, _I64, _I64, _I64, _P, _I64, _I64, _I64, _P]),
    "cg_decode_fast_prefsum": (_INT, [_P, _INT, _P, _I64, _P, _I64, _I64, _I64, _P, _I64, _I64, _I64, _P]),
    "cg_quantize_kv": (_INT, [_P, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P, _P, _P, _P, _P]),
    "cg_encode_kv_workspace": (_SZ, [_I64, _I64, _I64, _I64]),
    "cg_encode_kv": (_INT, [_P, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P, _P, _INT, _I64, _INT,
                            _P, _P, _P, _P, _P, _I64, _P, _P, _SZ, _P]),
    "cg_test_encode_kv": (_INT, [_P, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P, _P, _INT, _I64, _INT,
                                 _P, _P, _P, _P, _P, _I64, _P, _P, _SZ, _P, _INT]),
    "cg_encode_kv_levels_workspace": (_SZ, [_I64, _I64, _I64, _I64, _INT]),
    "cg_encode_kv_levels": (_INT, [_P, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _INT, _P, _P, _P, _I64,
                                   _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "cg_scan_workspace": (_SZ, [_I64]),
    "cg_scan_lengths": (_INT, [_P, _I64, _P, _P, _SZ, _P]),
    "cg_scan_lengths_static": (_INT, [_P, _I64, _P, _P]),
    "cg_tables_to_counts": (_INT, [_P, _INT, _I64, _I64, _P, _P, _P, _P, _P]),
    "cg_pack_counts": (_INT, [_P, _INT, _I64, _I64, _P, _P, _P, _P]),
    "cg_counts_to_tables": (_INT, [_P, _I64, _INT, _I64, _I64, _P, _P, _P, _P, _P, _P]),
    "cg_decode_kv": (_INT, [_P, _INT, _P, _INT, _P, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I64, _INT,
                            _P, _INT, _I64, _I64, _I64, _I64, _P]),
}

_handle = None


def library_path():
    return LIBRARY


def lib():
    """The loaded library; raises if it has not been built."""
    global _handle
    if _handle is None:
        if not os.path.exists(LIBRARY):
            raise RuntimeError(
                "cachegen_amd: %s is missing; build it with `python -m cachegen_amd.build` "
                "(hipcc, gfx950). There is no fallback path." % LIBRARY)
        h = ctypes.CDLL(LIBRARY)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(h, name)
            fn.restype = res
            fn.argtypes = args
        _handle = h
    return _handle


def check(rc):
    if rc != CG_OK:
        msg = lib().cg_last_error()
        raise RuntimeError(msg.decode() if msg else "cachegen_hip error %d" % rc)
