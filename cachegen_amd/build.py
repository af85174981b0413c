"""Build step of the HIP library: one hipcc line, output kept in-tree under lib/.

The two range coders are bound by the issue of vector instructions and need all eight
wavefronts that a SIMD can hold (five cost 17 % on the encoder): that is 64 vector registers a
lane and no scratch memory.  A compiler update or an edit that pushes a stream kernel past that
line costs a fifth of the throughput without failing any test, so the build reads the compiler's
own resource report for every kernel and fails when a budget below is broken.
"""
import json
import os
import re
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
SOURCE = os.path.join(_PKG, "csrc", "cachegen_hip.hip")
LIBRARY = os.path.join(_PKG, "lib", "libcachegen_hip.so")
RESOURCES = os.path.join(_PKG, "lib", "kernel_resources.json")
# the calibration probe bench.py prices the decoder's instruction count with (not part of the codec)
PROBE_SOURCE = os.path.join(_PKG, "csrc", "issue_probe.hip")
PROBE_LIBRARY = os.path.join(_PKG, "lib", "libcachegen_probe.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                     # float32 steps are rounded one by one
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Rpass-analysis=kernel-resource-usage", # per-kernel registers, scratch and occupancy, checked below
    "-I" + os.path.join(_ROOT, "include"),
]

# (pattern of the demangled kernel name, least wavefronts per SIMD).  Every kernel of the library
# must also run without scratch memory.
OCCUPANCY_BUDGETS = [
    (r"^encode_streams_kernel<", 7),         # the forms behind the four reference entry points and odd shapes
    (r"^encode_streams_kernel<256, true, true, (true|false), true, true>", 8),   # the fused path of cg_encode_kv
    (r"^decode_streams_kernel<", 8),
    (r"^compact_streams_kernel<", 8),
    (r"^quantize_pack_kernel<[01], (true|false), 2, false>", 8),                # up to 1024 channels, one level
    (r"^quantize_tables_kernel<[01], (true|false), [12], (9|17|33)>", 4),       # two blocks of eight wavefronts per compute unit
]


# Kernels that address their dynamically allocated LDS from byte 0 (the counters of the table
# builder: the address comes out of a byte permute): a statically allocated array would sit there.
NO_STATIC_LDS = r"^(quantize_tables_kernel|tables_from_partial_kernel)<"


def parse_kernel_resources(report):
    """{demangled kernel name: {"vgprs", "agprs", "sgprs", "scratch", "occupancy", "lds"}} from the
    remarks of -Rpass-analysis=kernel-resource-usage."""
    fields = {"VGPRs": "vgprs", "AGPRs": "agprs", "TotalSGPRs": "sgprs", "ScratchSize": "scratch",
              "Occupancy": "occupancy", "LDS Size": "lds"}
    mangled, cur = {}, None
    for line in report.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            cur = mangled.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+) \[-Rpass", line)
        if m and cur is not None and m.group(1).strip() in fields:
            cur[fields[m.group(1).strip()]] = int(m.group(2))
    if not mangled:
        return {}
    names = subprocess.run(["c++filt"], input="\n".join(mangled), stdout=subprocess.PIPE, text=True).stdout.splitlines()
    out = {}
    for name, res in zip(names, mangled.values()):
        name = name.replace("(anonymous namespace)::", "")
        name = re.sub(r"^void ", "", name).split("(")[0]
        out[name] = res
    return out


def check_budgets(resources):
    """Raises RuntimeError naming every kernel that uses scratch memory or holds fewer wavefronts
    per SIMD than its budget."""
    if not resources:
        raise RuntimeError("no kernel resource report: was the library built with -Rpass-analysis=kernel-resource-usage?")
    bad = []
    for name, r in sorted(resources.items()):
        if r.get("scratch", 0) != 0:
            bad.append("%s spills %d bytes per lane to scratch memory" % (name, r["scratch"]))
        if re.search(NO_STATIC_LDS, name) and r.get("lds", 0) != 0:
            bad.append("%s has %d bytes of statically allocated LDS: its counters are addressed from LDS byte 0" % (name, r["lds"]))
        need = max([n for pat, n in OCCUPANCY_BUDGETS if re.search(pat, name)] or [0])
        if r.get("occupancy", 0) < need:
            bad.append("%s: %d wavefronts per SIMD (%d vector registers), budget %d"
                       % (name, r.get("occupancy", 0), r.get("vgprs", -1), need))
    for pat, _ in OCCUPANCY_BUDGETS:
        if not any(re.search(pat, n) for n in resources):
            bad.append("no kernel matches the budget pattern %s" % pat)
    if bad:
        raise RuntimeError("kernel resource budget broken:\n  " + "\n  ".join(bad))


def build_library(verbose=False):
    """Compile csrc/cachegen_hip.hip for gfx950 into lib/libcachegen_hip.so, write the compiler's
    per-kernel resource figures beside it and check them against the budgets."""
    os.makedirs(os.path.dirname(LIBRARY), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIBRARY, SOURCE]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    resources = parse_kernel_resources(res.stdout)
    with open(RESOURCES, "w") as f:
        json.dump(resources, f, indent=0, sort_keys=True)
    if verbose:
        print("\n".join(l for l in res.stdout.splitlines() if "kernel-resource-usage" not in l))
    check_budgets(resources)
    return LIBRARY


def build_probe():
    """Compile csrc/issue_probe.hip into lib/libcachegen_probe.so."""
    os.makedirs(os.path.dirname(PROBE_LIBRARY), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", PROBE_LIBRARY, PROBE_SOURCE]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    return PROBE_LIBRARY


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_probe())
