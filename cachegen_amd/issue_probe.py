"""ctypes binding of lib/libcachegen_probe.so (csrc/issue_probe.hip): how fast a SIMD of this GPU
issues vector instructions and at which engine clock.  A measuring tool for bench.py and the
profiles, not part of the codec; nothing under serde/ or codec.py uses it."""
import ctypes

from .build import PROBE_LIBRARY

_handle = None

CHEAP, FULL, DECODER_SYMBOL = 0, 1, 2


def lib():
    global _handle
    if _handle is None:
        try:
            h = ctypes.CDLL(PROBE_LIBRARY)
        except OSError as e:
            raise RuntimeError("calibration probe not built (%s): run cachegen_amd.build.build_probe()" % e)
        h.cg_probe_issue_rate.restype = ctypes.c_int
        h.cg_probe_issue_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
        h.cg_probe_clock_start.restype = ctypes.c_int
        h.cg_probe_clock_start.argtypes = [ctypes.c_int, ctypes.c_void_p]
        h.cg_probe_clock_result.restype = ctypes.c_int
        h.cg_probe_clock_result.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
        _handle = h
    return _handle


def issue_rate(kind, iters=2048):
    """(ns per wave64 instruction per SIMD with 8 wavefronts resident, engine clock in MHz)."""
    ns, mhz = ctypes.c_double(), ctypes.c_double()
    rc = lib().cg_probe_issue_rate(kind, iters, ctypes.byref(ns), ctypes.byref(mhz))
    if rc:
        raise RuntimeError("cg_probe_issue_rate: hipError %d" % rc)
    return ns.value, mhz.value


def calibrate(iters=2048):
    """Cycles a SIMD takes per wave64 instruction of the cheap class, of the full-rate class and of
    the decoder's own instruction sequence, with the engine clock each was measured at."""
    out = {}
    for name, kind in (("cheap", CHEAP), ("full", FULL), ("decoder_symbol", DECODER_SYMBOL)):
        ns, mhz = issue_rate(kind, iters)
        out[name] = {"ns_per_instruction": round(ns, 4), "clock_mhz": round(mhz, 1), "cycles_per_instruction": round(ns * mhz * 1e-3, 3)}
    return out


def clock_window_start(microseconds, stream):
    """Queue the one-wavefront clock sampler on `stream` (a raw hipStream_t) for about that long."""
    rc = lib().cg_probe_clock_start(int(microseconds), ctypes.c_void_p(stream))
    if rc:
        raise RuntimeError("cg_probe_clock_start: hipError %d" % rc)


def clock_window_result():
    """(engine clock in MHz averaged over the sampler's window, window length in microseconds);
    call after the sampler's stream has been synchronized."""
    mhz, us = ctypes.c_double(), ctypes.c_double()
    rc = lib().cg_probe_clock_result(ctypes.byref(mhz), ctypes.byref(us))
    if rc:
        raise RuntimeError("cg_probe_clock_result: hipError %d" % rc)
    return mhz.value, us.value


if __name__ == "__main__":
    import json
    print(json.dumps(calibrate(), indent=1))
