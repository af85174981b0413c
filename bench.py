#!/usr/bin/env python3
"""Benchmark of the KV codec hot path on one MI355X.

A step is one encode of the whole synthetic KV cache followed by one decode of the
result, inputs and outputs resident in HBM, every buffer allocated before the timed
region.  Prints ONE JSON line.  Workload (default, "config2"): a Mistral-7B-shape
cache, 32 layers x {K,V} x 8192 tokens x 8 heads x 128, fp16, one
table per 256-token chunk, reference 7B bins table.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    # name: (layers, tokens, heads, head_size, chunk_tokens, model name for the bins table, seed)
    "config1": (2, 512, 8, 64, 512, None, 1235),
    "config2": (32, 8192, 8, 128, 256, "mistralai/Mistral-7B-Instruct-v0.2", 1236),
    "config2_small": (32, 1024, 8, 128, 256, "mistralai/Mistral-7B-Instruct-v0.2", 1236),
    # the reference's own call: run_cachegen.py:53,67 hands the serializer the whole context as one
    # chunk, so one table per (layer, channel) covers all 8192 tokens and their 32 sub-chunks
    "config2_one_table": (32, 8192, 8, 128, 8192, "mistralai/Mistral-7B-Instruct-v0.2", 1236),
    "config3": (32, 16384, 32, 128, 256, "mistralai/Mistral-7B-Instruct-v0.2", 1237),
    "config4": (80, 32768, 8, 128, 1500, "Yukang/LongAlpaca-70B-16k", 1238),
    "config5": (32, 4096, 8, 128, 256, "levels", 1239),
}

# config 5: four quantization levels over the 32-layer tiers (first 10 / next 10 / rest for K,
# first 2 / rest for V): A = 8 bins everywhere, B = reference QUANT_LEVEL 1, C = reference
# QUANT_LEVEL 2, D = 64/32/32 and 64/32 (wider than the reference's tables allow).
CONFIG5_LEVELS = {
    "A": ((8, 8, 8), (8, 8)),
    "B": ((16, 16, 12), (16, 12)),
    "C": ((32, 16, 16), (32, 16)),
    "D": ((64, 32, 32), (64, 32)),
}


def bins_for(name, model, layers):
    import torch
    from cachegen_amd.serde import cachegen_basics as B
    if model is None:        # config 1: 32 bins for the first half of the layers, 16 for the rest
        k = torch.tensor([32.0] * (layers // 2) + [16.0] * (layers - layers // 2))
        return k, k.clone()
    os.environ.setdefault("QUANT_LEVEL", "2")
    cfg = B.CacheGenConfig.from_model_name(model)
    return B.make_key_bins(cfg), B.make_value_bins(cfg)


def run_levels(args, quiet=False):
    """config 5: the same cache encoded at four levels from one read of the tensor
    (cg_encode_kv_levels), next to four separate encodes; decode per level.  One JSON line."""
    import torch
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv
    from cachegen_amd.serde import cachegen_basics as B
    L, T, H, D, chunk, _, seed = WORKLOADS["config5"]
    dev = torch.device("cuda:0")
    rho = [0.5 if l % 2 == 0 else 0.95 for l in range(L)]      # even layers rho 0.5, odd 0.95
    kv = make_kv(L, T, H, D, seed=seed, rho=rho, device=dev)
    C = H * D
    names = list(CONFIG5_LEVELS)
    levels, max_bins = [], []
    for name in names:
        kt, vt = CONFIG5_LEVELS[name]
        cfg = B.CacheGenConfig.from_layer_tiers(L, [(10, kt[0]), (20, kt[1]), kt[2]], [(2, vt[0]), vt[1]])
        levels.append((B.make_key_bins(cfg).to(dev), B.make_value_bins(cfg).to(dev)))
        max_bins.append(int(max(kt + vt)))
    workspace = torch.empty(codec.encode_levels_workspace_bytes(L, T, C, chunk, len(names)), dtype=torch.uint8, device=dev)
    out = torch.empty((L, 2, T, H, D), dtype=torch.float16, device=dev)
    kv_bytes = kv.numel() * 2

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    encs = codec.encode_kv_levels(kv, levels, chunk_tokens=chunk, max_bins=max_bins, workspace=workspace)
    for e in encs:
        e.check()
    # untimed repetitions until the GPU has reached its running clock (see run_workload)
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < getattr(args, "clock_ramp_ms", 60.0):
        codec.encode_kv_levels(kv, levels, chunk_tokens=chunk, max_bins=max_bins, workspace=workspace, out=encs)
        torch.cuda.synchronize()
    together_ms = timed(lambda: codec.encode_kv_levels(kv, levels, chunk_tokens=chunk, max_bins=max_bins,
                                                       workspace=workspace, out=encs))
    rows = {}
    separate_ms = decode_ms = 0.0
    for name, (kb, vb), mb, enc in zip(names, levels, max_bins, encs):
        single = codec.encode_kv(kv, kb, vb, chunk_tokens=chunk, max_bins=mb, workspace=workspace)
        n = enc.total_bytes()
        same = bool(single.total_bytes() == n and torch.equal(single.payload[:n], enc.payload[:n])
                    and torch.equal(single.cdf, enc.cdf) and torch.equal(single.lengths, enc.lengths))
        e_ms = timed(lambda: codec.encode_kv(kv, kb, vb, chunk_tokens=chunk, max_bins=mb, workspace=workspace, out=single))
        d_ms = timed(lambda: codec.decode_encoded(enc, kb, vb, fmt="vllm", out=out))
        separate_ms += e_ms
        decode_ms += d_ms
        side = 2 * (mb + 1) * 2 * L * C * enc.num_chunks + 4 * enc.lengths.numel() + 2 * 2 * L * T
        kt, vt = CONFIG5_LEVELS[name]
        rows[name] = {"bins": {"key": kt, "value": vt}, "encode_alone_GBps": round(kv_bytes / e_ms / 1e6, 2),
                      "decode_GBps": round(kv_bytes / d_ms / 1e6, 2),
                      "compression_ratio_payload": round(kv_bytes / n, 3),
                      "compression_ratio_total": round(kv_bytes / (n + side), 3),
                      "identical_to_separate_encode": same}
    t_all = together_ms + decode_ms
    result = {
        "metric": "KV encode & decode GB/s (fp16 input) + % HBM roofline + compression ratio",
        "value": round(2 * 4 * kv_bytes / (t_all * 1e-3) / 1e9, 3), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(t_all, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": "config5: 32 layers x {K,V} x 4096 tokens x 8 heads x 128, fp16, table per 256 tokens, "
                               "four quantization levels, AR(1) rho 0.5 (even layers) / 0.95 (odd layers), seed %d" % seed,
                   "value_is": "fp16 KV bytes of four encodes (one pass over the tensor) plus four decodes, per second"},
        "encode_four_levels_at_once_ms": round(together_ms, 4),
        "encode_four_levels_separately_ms": round(separate_ms, 4),
        "encode_at_once_GBps_per_level": round(4 * kv_bytes / together_ms / 1e6, 2),
        "decode_four_levels_ms": round(decode_ms, 4),
        "levels": rows}
    if not quiet:
        print(json.dumps(result))
    return result


def algorithmic_bytes(L, T, C, lp, nchunks, nstreams, payload):
    """Bytes that must cross HBM: the 16-bit tensor once, the compact payload once, the tables,
    one int32 length per stream and the row maxima."""
    n = 2 * L * T * C
    side = 2 * lp * (2 * L * C) * nchunks + 4 * nstreams + 2 * 2 * L * T
    return dict(kv=2 * n, side=side, payload=payload, encode=2 * n + payload + side,
                decode=2 * n + payload + side)


def measured_counters():
    """Per-launch counter readings of the committed rocprofv3 profiles (profiles/*.txt), kept as
    numbers in profiles/measured_counters.json: they are measurements of a profiled run of this
    script, not something it can observe while it runs."""
    path = os.path.join(ROOT, "profiles", "measured_counters.json")
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        return json.load(f)


# --encode-form: the library's internal forms of the encode call, forced through its test entry
# point (cg_test_encode_kv); the results are the same bytes, the profiles compare their cost
ENCODE_FORMS = {"default": None, "tables-in-quantizer": 2, "tables-in-coder": 4, "byte-symbols": 1,
                "tables-in-coder+byte-symbols": 5, "chunks-in-parts": 2 | 8}


def run_workload(name, steps, warmup, fmt="vllm", copy_probe=False, keep=False, ramp_ms=0.0, sample_clock=False,
                 encode_form="default"):
    """Encode + decode of one workload, timed with HIP events on the launching stream.
    Returns a dict of figures (and, with keep=True, the tensors for further use)."""
    import torch
    from cachegen_amd import codec
    from cachegen_amd.kvgen import make_kv

    L, T, H, D, chunk, model, seed = WORKLOADS[name]
    C = H * D
    dev = torch.device("cuda:0")
    kbins, vbins = bins_for(name, model, L)
    kv = make_kv(L, T, H, D, seed=seed, device=dev)
    if fmt == "huggingface":
        kv = kv.permute(0, 1, 3, 2, 4).contiguous()
    kb, vb = kbins.to(dev), vbins.to(dev)
    max_bins = int(max(kbins.max(), vbins.max()))

    workspace = torch.empty(codec.encode_workspace_bytes(L, T, C, chunk), dtype=torch.uint8, device=dev)
    flags = ENCODE_FORMS[encode_form]
    enc = codec.encode_kv(kv, kb, vb, chunk_tokens=chunk, max_bins=max_bins, workspace=workspace, fmt=fmt, _test_flags=flags)
    # bit 0: a stream outgrew its 256 bytes and was cut (possible only when a table covers many
    # more tokens than a stream holds); reported, and then the round trip is not checked
    status = int(enc.status.item())
    if status & ~1:
        enc.check()
    out = torch.empty_like(kv)

    def encode():
        codec.encode_kv(kv, kb, vb, chunk_tokens=chunk, max_bins=max_bins, workspace=workspace, out=enc, fmt=fmt, _test_flags=flags)

    def decode():
        codec.decode_encoded(enc, kb, vb, fmt=fmt, out=out)

    # The GPU idles at a low clock and takes tens of milliseconds of work to reach its running
    # clock (with 3 warm-up steps, about 5 ms, the timed steps read 7-10 % slower than after 20):
    # the same step is repeated, untimed, for ramp_ms before the warm-up steps proper.
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < ramp_ms:
        encode()
        decode()
        torch.cuda.synchronize()
    for _ in range(warmup):
        encode()
        decode()
    torch.cuda.synchronize()

    # per-phase device times: HIP events on the stream the kernels are queued on
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i][0].record()
        encode()
        ev[i][1].record()
        decode()                      # a single launch of decode_streams_kernel
        ev[i][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    clock = None
    if sample_clock:
        # The engine clock these steps run at: the same steps once more, untimed, with one idle
        # wavefront on a side stream that reads the shader clock against the 100 MHz counter over
        # their whole length.  (Not during the timed steps: a resident wavefront leaves its SIMD one
        # slot short, and that compute unit's blocks then hold up the end of every launch: +2 to 4 %.)
        from cachegen_amd import issue_probe
        side = torch.cuda.Stream()
        issue_probe.clock_window_start(max(200, int(0.9 * wall * 1e6)), side.cuda_stream)
        for i in range(steps):
            encode()
            decode()
        torch.cuda.synchronize()
        mhz, window_us = issue_probe.clock_window_result()
        clock = {"engine_clock_mhz": round(mhz, 1), "window_us": round(window_us, 1),
                 "what": "average over a repetition of the timed steps (%d steps, %.1f ms)" % (steps, wall * 1e3)}

    enc_ms = sorted(e[0].elapsed_time(e[1]) for e in ev)
    dec_ms = sorted(e[1].elapsed_time(e[2]) for e in ev)
    enc_avg = sum(enc_ms) / len(enc_ms)
    dec_avg = sum(dec_ms) / len(dec_ms)

    if copy_probe:
        out.copy_(kv)                 # reads and writes kv_bytes each: the known-size reference kernel
        torch.cuda.synchronize()
        decode()
        torch.cuda.synchronize()

    payload = enc.total_bytes()
    nstreams = enc.lengths.numel()
    ab = algorithmic_bytes(L, T, C, max_bins + 1, enc.num_chunks, nstreams, payload)
    kv_bytes = ab["kv"]

    # round trip must reconstruct within half a quantization step of every row
    # (half a step plus the 16-bit rounding of the output), checked in slices of layers
    maxq = torch.stack([kb, vb], dim=1).div(2, rounding_mode="floor").sub(1)[:, :, None, None]
    verified = True
    group = 8 if C <= 1024 else 4
    for l0 in range(0, L if not status else 0, group):
        xs, ys = kv[l0:l0 + group], out[l0:l0 + group]
        if fmt == "huggingface":
            xs, ys = xs.permute(0, 1, 3, 2, 4), ys.permute(0, 1, 3, 2, 4)
        x = xs.reshape(-1, 2, T, C).float()
        y = ys.reshape(-1, 2, T, C).float()
        step = x.abs().amax(dim=-1, keepdim=True) / maxq[l0:l0 + group]
        verified = verified and bool(((x - y).abs() <= 0.52 * step).all())
        del x, y, step

    r = {
        "workload": "%s: %d layers x {K,V} x %d tokens x %d heads x %d, fp16, one table per %d tokens, "
                    "AR(1) rho=0.9 lognormal-channel generator seed %d%s"
                    % (name, L, T, H, D, chunk, seed, "" if fmt == "vllm" else ", layout [L,2,H,T,D]"),
        "kv_bytes": kv_bytes, "streams": nstreams, "wall_ms_per_step": wall * 1000.0 / steps,
        "encode_ms": enc_avg, "decode_ms": dec_avg,
        "encode_ms_median": enc_ms[len(enc_ms) // 2], "decode_ms_median": dec_ms[len(dec_ms) // 2],
        "encode_GBps": kv_bytes / (enc_avg * 1e-3) / 1e9, "decode_GBps": kv_bytes / (dec_avg * 1e-3) / 1e9,
        "encode_roofline_frac": ab["encode"] / (enc_avg * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "decode_roofline_frac": ab["decode"] / (dec_avg * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "compression_ratio_payload": kv_bytes / payload,
        "compression_ratio_total": kv_bytes / (payload + ab["side"]),
        "payload_bytes": payload, "algorithmic_bytes": ab,
        "round_trip_within_half_step": verified if not status else None,
        "streams_cut_at_256_bytes": bool(status & 1), "longest_stream_bytes": int(enc.lengths.max().item()),
        "clock": clock,
    }
    if 256 < chunk < T:
        # streaming case: latency of decoding one chunk on its own
        tdim = 2 if fmt == "vllm" else 3
        one = codec.encode_kv(kv.narrow(tdim, 0, chunk), kb, vb, chunk_tokens=chunk, max_bins=max_bins, fmt=fmt)
        one_out = torch.empty_like(kv.narrow(tdim, 0, chunk))
        for _ in range(3):
            codec.decode_encoded(one, kb, vb, fmt=fmt, out=one_out)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            codec.decode_encoded(one, kb, vb, fmt=fmt, out=one_out)
        e1.record()
        torch.cuda.synchronize()
        r["decode_ms_per_%d_token_chunk" % chunk] = e0.elapsed_time(e1) / 10
        del one, one_out
    if keep:
        r["_keep"] = dict(kv=kv, enc=enc, kbins=kbins, vbins=vbins, chunk=chunk, L=L, T=T, C=C)
    else:
        del kv, out, enc, workspace
        torch.cuda.empty_cache()
    return r


def other_config_summary(r):
    """The figures of a secondary workload that go into the main JSON line."""
    keys = ["encode_ms", "decode_ms", "encode_GBps", "decode_GBps", "encode_roofline_frac", "decode_roofline_frac",
            "compression_ratio_payload", "compression_ratio_total", "round_trip_within_half_step",
            "streams_cut_at_256_bytes", "longest_stream_bytes"]
    out = {"workload": r["workload"]}
    for k in keys:
        out[k] = round(r[k], 4) if isinstance(r[k], float) else r[k]
    for k in r:
        if k.startswith("decode_ms_per_"):
            out[k] = round(r[k], 4)
    return out


def cpu_baseline(kv_cpu, kbins, vbins, chunk, sample_tokens):
    """The CPU path beside the GPU figures: PyTorch-CPU quantization and dequantization (the tensor
    code of cachegen_encoder.py:42-59 and cachegen_decoder.py:24-34, on torch's own thread pool)
    around the C oracle's table builder and arithmetic coder (OpenMP over streams), on the first
    `sample_tokens` tokens, one `to_bytes`-sized chunk at a time."""
    import numpy as np
    import torch
    from oracle import cachegen_oracle as oracle
    L, _, T, H, D = kv_cpu.shape
    C = H * D
    n = min(sample_tokens, T)
    oracle.lib()
    cores = oracle.max_threads()
    torch.set_num_threads(cores)
    maxq = torch.stack([kbins, vbins], dim=1).to(torch.float32).div(2, rounding_mode="floor").sub(1)[:, :, None, None]

    def quantize(x):                     # x: [L, 2, n, C] 16-bit floats
        max1 = x.abs().amax(dim=-1, keepdim=True)
        factor = maxq / max1
        sym = torch.round(x * factor + maxq).to(torch.int8)
        return sym, max1

    def dequantize(sym, max1, dtype):    # sym: uint8 [L, 2, n, C]
        return (((sym.float() - maxq) / maxq) * max1).to(dtype)

    def encode(x):
        sym, max1 = quantize(x)
        s = np.ascontiguousarray(sym.permute(1, 0, 2, 3).reshape(2 * L, x.shape[2], C).numpy().view(np.uint8))
        cdf = oracle.calculate_cdf(s, int(max(kbins.max(), vbins.max())))
        subs = []
        for t0 in range(0, s.shape[1], 256):
            padded, lengths = oracle.encode_fast_new(cdf, s[:, t0:t0 + 256])
            subs.append((oracle.collect_bytes(padded, lengths), lengths, min(256, s.shape[1] - t0)))
        return cdf, max1, subs, s

    def decode(cdf, max1, subs, dtype):
        nt = sum(k for _, _, k in subs)
        sym = np.zeros((2 * L, nt, C), dtype=np.uint8)
        t0 = 0
        for data, lengths, k in subs:
            prefix = lengths.astype(np.int64).ravel().cumsum().reshape(lengths.shape)
            oracle.decode_fast_prefsum(cdf, data, prefix, k, sym[:, t0:t0 + k])
            t0 += k
        return sym, dequantize(torch.from_numpy(sym).view(2, L, nt, C).permute(1, 0, 2, 3), max1, dtype)

    x = kv_cpu[:, :, :n].reshape(L, 2, n, C)
    t0 = time.perf_counter()
    encs = [encode(x[:, :, s:min(s + chunk, n)]) for s in range(0, n, chunk)]
    t1 = time.perf_counter()
    ok = True
    for cdf, max1, subs, s in encs:
        back, _ = decode(cdf, max1, subs, x.dtype)
        ok = ok and np.array_equal(back, s)
    t2 = time.perf_counter()
    nbytes = 2 * L * n * C * 2
    # the same code on one core, on the first chunk only
    one = x[:, :, :min(chunk, n)]
    oracle.set_threads(1)
    torch.set_num_threads(1)
    s0 = time.perf_counter()
    decode(*encode(one)[:3], x.dtype)
    s1 = time.perf_counter()
    oracle.set_threads(cores)
    torch.set_num_threads(cores)
    one_bytes = 2 * L * one.shape[2] * C * 2
    return dict(value=round(2 * nbytes / (t2 - t0) / 1e9, 4), unit="GB/s", cores=cores, kind="port",
                sample="first %d tokens of the workload (%d chunks of %d): %.1f MB fp16; PyTorch-CPU quantization and "
                       "dequantization, C restatement of the table builder and coder with OpenMP over streams"
                       % (n, len(encs), chunk, nbytes / 1e6),
                encode_GBps=round(nbytes / (t1 - t0) / 1e9, 4), decode_GBps=round(nbytes / (t2 - t1) / 1e9, 4),
                round_trip_symbols_equal=bool(ok),
                one_core_GBps=round(2 * one_bytes / (s1 - s0) / 1e9, 4),
                one_core_sample="first chunk (%d tokens, %.1f MB fp16)" % (one.shape[2], one_bytes / 1e6))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--clock-ramp-ms", type=float, default=60.0,
                    help="untimed repetitions of the step before the warm-up steps, until the GPU has reached its running clock")
    ap.add_argument("--workload", default="config2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of configs 3, 4 and 5 that the default workload appends")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192)
    ap.add_argument("--fmt", default="vllm", choices=["vllm", "huggingface"],
                    help="layout of the KV tensor: [L,2,T,H,D] (vllm, the metric's layout) or [L,2,H,T,D]")
    ap.add_argument("--encode-form", default="default", choices=sorted(ENCODE_FORMS),
                    help="force one of the library's internal forms of the encode call (same bytes; for profiles)")
    ap.add_argument("--no-issue-probe", action="store_true",
                    help="skip the engine-clock sampler and the instruction-issue calibration (valu_issue)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain device copy of the KV tensor (calibrates rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this codec runs on one GPU; --gpus must be 1 (the path shards by layer or by "
              "token chunk with no exchange)", file=sys.stderr)
        sys.exit(2)

    if args.workload == "config5":
        run_levels(args)
        return

    import torch
    torch.cuda.set_device(0)
    fmt = args.fmt
    r = run_workload(args.workload, args.steps, args.warmup, fmt=fmt, copy_probe=args.copy_probe, keep=True,
                     ramp_ms=args.clock_ramp_ms, sample_clock=not args.no_issue_probe, encode_form=args.encode_form)
    kept = r.pop("_keep")
    ab = r["algorithmic_bytes"]
    kv_bytes = r["kv_bytes"]
    ms_per_step = r["wall_ms_per_step"]
    counters = measured_counters().get(args.workload, {}).get("decode_streams_kernel", {})
    traffic = counters.get("fetch_bytes", 0) + counters.get("write_bytes", 0)

    result = {
        "metric": "KV encode & decode GB/s (fp16 input) + % HBM roofline + compression ratio",
        "value": round(2 * kv_bytes / (ms_per_step * 1e-3) / 1e9, 3),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_ramp_ms": args.clock_ramp_ms,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {
            "workload": r["workload"],
            "value_is": "fp16 KV bytes encoded plus decoded per second of a full encode+decode step",
            "kv_bytes": kv_bytes,
            "streams": r["streams"],
            **({"encode_form": args.encode_form} if args.encode_form != "default" else {}),
        },
        "encode_GBps": round(r["encode_GBps"], 3),
        "decode_GBps": round(r["decode_GBps"], 3),
        "encode_ms": round(r["encode_ms"], 4),
        "decode_ms": round(r["decode_ms"], 4),
        "encode_ms_median": round(r["encode_ms_median"], 4),
        "decode_ms_median": round(r["decode_ms_median"], 4),
        "encode_roofline_frac": round(r["encode_roofline_frac"], 4),
        "decode_roofline_frac": round(r["decode_roofline_frac"], 4),
        "compression_ratio_payload": round(r["compression_ratio_payload"], 3),
        "compression_ratio_total": round(r["compression_ratio_total"], 3),
        "payload_bytes": r["payload_bytes"],
        "round_trip_within_half_step": r["round_trip_within_half_step"],
        "roofline": {
            "kernel": "decode_streams_kernel",
            "bound": "hbm",
            "achieved": round(ab["decode"] / (r["decode_ms"] * 1e-3) / 1e9, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(r["decode_roofline_frac"], 4),
            "traffic": traffic if traffic else None,       # profiles/measured_counters.json; null = not profiled
            "algorithmic_bytes": ab["decode"],
            "avg_launch_ms": round(r["decode_ms"], 4),
        },
    }
    if "valu_insts" in counters and not args.no_issue_probe:
        # The decoder's own limit is the issue of vector instructions.  Its instruction count per
        # launch (the committed profile's SQ_INSTS_VALU) is priced with what this GPU issues, measured
        # now by the calibration probe (cachegen_amd/csrc/issue_probe.hip): cycles per wave64
        # instruction of the cheap class (adds, logic, right shifts, moves, float add/multiply on
        # registers) and of all others, at the engine clock sampled while the timed steps ran.
        from cachegen_amd import issue_probe
        cal = issue_probe.calibrate()
        insts = counters["valu_insts"]
        cheap = counters.get("cheap_class_fraction", 11.0 / 38.0)
        simds = torch.cuda.get_device_properties(0).multi_processor_count * 4
        mhz = (r.get("clock") or {}).get("engine_clock_mhz") or cal["decoder_symbol"]["clock_mhz"]
        per_simd = insts / simds
        two_class = cheap * cal["cheap"]["cycles_per_instruction"] + (1.0 - cheap) * cal["full"]["cycles_per_instruction"]
        bound_ms = per_simd * two_class / (mhz * 1e3)
        seq_ms = per_simd * cal["decoder_symbol"]["cycles_per_instruction"] / (mhz * 1e3)
        result["valu_issue"] = {
            "kernel": "decode_streams_kernel",
            "insts_per_launch": insts,
            "insts_per_symbol_and_lane": round(insts * 64 / (kv_bytes / 2), 1),
            "cheap_class_fraction": round(cheap, 3),
            "calibration": cal,
            "engine_clock_mhz_during_timed_steps": mhz,
            "issue_time_ms_two_class": round(bound_ms, 4),
            "frac_of_issue_rate": round(bound_ms / r["decode_ms"], 3),
            "issue_time_ms_same_sequence_in_probe": round(seq_ms, 4),
            "frac_of_probe_sequence_rate": round(seq_ms / r["decode_ms"], 3),
            "note": "instruction count of the committed profile x cycles per instruction measured now by the probe "
                    "(two classes; and the decoder's own symbol sequence issued from the probe) / engine clock "
                    "sampled during the timed steps / live decode time",
        }
    if r.get("clock"):
        result["clock"] = r["clock"]
    enc_counters = measured_counters().get(args.workload, {}).get("encode_all_kernels")
    if enc_counters:
        result["encode_traffic"] = {
            "bytes": enc_counters["fetch_bytes"] + enc_counters["write_bytes"], "algorithmic_bytes": ab["encode"],
            "ratio": round((enc_counters["fetch_bytes"] + enc_counters["write_bytes"]) / ab["encode"], 2),
            "source": enc_counters["source"]}
    for k in r:
        if k.startswith("decode_ms_per_"):
            result[k] = round(r[k], 4)
    # what one chunk weighs on the wire in the two flat containers (first chunk, vllm layout only)
    if fmt == "vllm":
        from cachegen_amd.serde import wire
        enc = kept["enc"]
        flat_blob = wire.pack_chunks(enc, 0, 1)[0]
        compact_blob = wire.pack_chunks(enc, 0, 1, compact=True)[0]
        chunk_fp16 = 2 * kept["L"] * min(kept["chunk"], kept["T"]) * kept["C"] * 2
        result["first_chunk_container"] = {
            "fp16_bytes": chunk_fp16, "flat_bytes": len(flat_blob), "compact_bytes": len(compact_blob),
            "ratio_flat": round(chunk_fp16 / len(flat_blob), 3), "ratio_compact": round(chunk_fp16 / len(compact_blob), 3)}
    if not args.no_cpu_baseline:
        kv = kept["kv"]
        kv_vllm = kv if fmt == "vllm" else kv.permute(0, 1, 3, 2, 4)
        result["cpu_baseline"] = cpu_baseline(kv_vllm[:, :, :args.cpu_sample_tokens].cpu(), kept["kbins"], kept["vbins"],
                                              kept["chunk"], args.cpu_sample_tokens)
    del kept
    torch.cuda.empty_cache()
    if args.workload == "config2" and fmt == "vllm" and not args.no_other_configs:
        # the other benchmark configurations, a few steps each, so that their figures are observed
        # by whoever runs this script and not only quoted
        others = {}
        for name in ("config2_one_table", "config3", "config4"):
            others[name] = other_config_summary(run_workload(name, max(2, min(args.steps, 5)), 1, ramp_ms=args.clock_ramp_ms))
        lv = run_levels(argparse.Namespace(steps=max(2, min(args.steps, 5)), warmup=1, clock_ramp_ms=args.clock_ramp_ms), quiet=True)
        others["config5"] = {k: lv[k] for k in ("config", "encode_four_levels_at_once_ms", "encode_four_levels_separately_ms",
                                                "encode_at_once_GBps_per_level", "decode_four_levels_ms", "levels")}
        result["other_configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
