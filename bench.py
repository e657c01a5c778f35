#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]

The headline workload is the radix sort of 2^28 uniform uint32 keys
(ascending).  A "step" is one sort of the full array; the unsorted input is
restored from a resident copy before each step, outside the timed intervals,
so every step sorts the same data with inputs already in HBM.  The last line
printed is one JSON object with the throughput, the roofline figure of the
dominant kernel (from per-kernel HIP events recorded by the library) and the
CPU path timed on a bounded sample.  The other primitives are measured the
same way and reported under "other_workloads".
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--log2n", type=int, default=28,
                   help="log2 of the key count of the headline sort")
    p.add_argument("--no-extras", action="store_true",
                   help="skip the other primitives")
    p.add_argument("--no-cpu", action="store_true",
                   help="skip the CPU baseline")
    p.add_argument("--cpu-log2n", type=int, default=27,
                   help="log2 of the CPU baseline sample size")
    p.add_argument("--short-sorts", action="store_true",
                   help="instead of the benchmark: sorts of 2^15 to 2^23 keys with and "
                        "without short tiles, one JSON line")
    return p.parse_args()


class Timer:
    """Times `fn` per step with HIP events on torch's current stream (the
    stream the library launches on), excluding the untimed `prepare`."""

    def __init__(self, torch):
        self.torch = torch

    def run(self, prepare, fn, steps, warmup):
        torch = self.torch
        for _ in range(warmup):
            prepare()
            fn()
        torch.cuda.synchronize()
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        wall0 = time.perf_counter()
        for i in range(steps):
            prepare()
            starts[i].record()
            fn()
            stops[i].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
        ms = [s.elapsed_time(e) for s, e in zip(starts, stops)]
        return ms, wall


def short_sorts(torch, capi, datagen, timer, wrap, steps, warmup):
    """Whole sorts of short inputs (keys without values) in the tile class they
    take by default against full tiles (the library's test hook switches the
    short classes off): median ms per sort, one JSON line."""
    rows = {}
    for name, dtype, sizes in (
            ("u32", np.uint32, [1 << 15, 1 << 16, 1 << 17, 1 << 18, 1 << 19, 1 << 20, 1 << 21,
                                3 << 20, 1 << 22, 5 << 20, 1 << 23]),
            ("u64", np.uint64, [1 << 15, 1 << 16, 1 << 17, 1 << 18, 1 << 19, 1 << 20])):
        for m in sizes:
            if dtype == np.uint32:
                part = datagen.uniform_u32_torch(m)
            else:
                part = datagen.splitmix64_torch(m)
            wk = torch.empty_like(part)
            kv = wrap(wk, dtype)
            tp = capi.temp_buffer(capi.radix_sort_temp_bytes(m, dtype))
            entry = {}
            for label, limit in (("full_tiles_ms", 0), ("default_ms", -1)):
                capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, limit)
                ms, _ = timer.run(lambda: wk.copy_(part), lambda: capi.radix_sort_keys(kv, tp),
                                  steps, warmup)
                entry[label] = round(float(np.median(ms)), 4)
            capi.sort_set_parameter(capi.SORT_PARAM_SHORT_TILE_MAX_TILES, -1)
            # unsigned order through signed compares: low 32 bits widened, or
            # the 64 bits with the sign bit flipped
            srt = wk.to(torch.int64) & 0xFFFFFFFF if dtype == np.uint32 else wk ^ (-1 << 63)
            entry["sorted"] = bool((srt[1:] >= srt[:-1]).all().item())
            rows[f"{name}_{m}"] = entry
            log(f"[bench] short sort {name} n={m}: full tiles {entry['full_tiles_ms']} ms, "
                f"default {entry['default_ms']} ms")
    print(json.dumps({"short_sorts": rows}))


def kernel_stats(capi, name):
    launches, total_ms = capi.profile_query(name)
    return launches, (total_ms / launches if launches else 0.0)


# HBM bytes per launch of each workload's dominant kernel come from rocprofv3
# counter runs of this script (FETCH_SIZE and WRITE_SIZE in separate runs, each
# scaled by what the same counter reads for a 1 GiB device copy).  A counter
# run cannot be nested inside this script, so the figures are kept in
# profiles/hbm_traffic.json together with the SHA-256 of the kernel source they
# were measured on; a figure whose source has changed since is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
CSRC = os.path.join(ROOT, "ilgpu_amd", "csrc")


def source_digest(file_name):
    """Digest of what a kernel is built from: the code of its source file and of
    the headers every kernel file includes, and the compiler flags.  // comments,
    indentation and blank lines do not count, so that only a change of code (or
    of the build) makes the counters stale."""
    import hashlib
    from ilgpu_amd import build
    lines = list(build.FLAGS)
    for name in (file_name, "common.hpp", "kernels.hpp"):
        if name != file_name and not os.path.exists(os.path.join(CSRC, name)):
            continue
        with open(os.path.join(CSRC, name), encoding="utf-8") as f:
            for line in f:
                code = line.split("//", 1)[0].strip()
                if code:
                    lines.append(code)
    return hashlib.sha256("\n".join(lines).encode()).hexdigest()[:16]


def measured_traffic(workload, default_size):
    """(bytes per launch or None, provenance) for a bench workload."""
    if not default_size or not os.path.exists(TRAFFIC_FILE):
        return None, None
    with open(TRAFFIC_FILE) as f:
        table = json.load(f)
    entry = table.get("workloads", {}).get(workload)
    if entry is None:
        return None, None
    source = {"file": "profiles/hbm_traffic.json", "kernel_source": entry["source"],
              "measured_on_sha256": entry["sha256"]}
    if source_digest(entry["source"]) != entry["sha256"]:
        source["stale"] = "kernel source changed since the counters were read"
        return None, source
    return entry["bytes_per_launch"], source


def roofline(achieved_gbs, traffic=None, traffic_source=None):
    r = {"bound": "hbm", "achieved": round(achieved_gbs, 1),
         "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(achieved_gbs / HBM_PEAK_GBS, 4), "traffic": traffic}
    if traffic_source is not None:
        r["traffic_source"] = traffic_source
    return r


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported "
              "(this build has no multi-GPU path)", file=sys.stderr)
        sys.exit(2)

    import torch
    from ilgpu_amd import capi, datagen

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    capi.lib()  # fails loudly if the HIP library is missing
    torch.cuda.set_device(0)
    D = capi.DeviceArray
    timer = Timer(torch)
    K, W = args.steps, args.warmup

    def wrap(t, dtype):
        """A DeviceArray over the memory of a torch tensor."""
        b = t.view(torch.uint8).reshape(-1)
        return D(b.numel() // np.dtype(dtype).itemsize, dtype, _bytes=b)

    if args.short_sorts:
        short_sorts(torch, capi, datagen, timer, wrap, max(K, 40), max(W, 5))
        return

    # ------------------------------------------------------------ headline
    n = 1 << args.log2n
    log(f"[bench] generating 2^{args.log2n} uniform uint32 keys on the GPU")
    src = datagen.uniform_u32_torch(n)
    work = torch.empty_like(src)
    keys = wrap(work, np.uint32)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n, np.uint32))

    def restore():
        work.copy_(src)

    def sort():
        capi.radix_sort_keys(keys, temp)

    log(f"[bench] radix sort: {W} warm-up + {K} timed steps")
    ms, wall = timer.run(restore, sort, K, W)
    ms_per_step = float(np.median(ms))   # median of the K timed steps
    mean_ms_per_step = float(np.mean(ms))
    gkeys = n / (ms_per_step * 1e-3) / 1e9

    # Same K steps again with the library's per-kernel event timing enabled.
    capi.profile_enable(True)
    timer.run(restore, sort, K, 0)
    pass_launches, pass_ms = kernel_stats(capi, "sort_onesweep")
    hist_launches, hist_ms = kernel_stats(capi, "sort_histogram")
    kernel_ms = {name: round(kernel_stats(capi, name)[1], 4) for name in
                 ("zero_words", "sort_histogram", "sort_plan", "sort_onesweep",
                  "sort_finish")}
    capi.profile_enable(False)
    passes, _ = capi.radix_sort_passes(temp, n, np.uint32)   # executed, from the sort's plan
    pass_bytes = 2.0 * n * 4            # read + write of the keys, one pass
    pass_gbs = pass_bytes / (pass_ms * 1e-3) / 1e9 if pass_ms else 0.0
    sort_bytes = n * 4.0 * (2 * passes + 1)
    sort_gbs = sort_bytes / (ms_per_step * 1e-3) / 1e9

    # Cheap verification on the GPU: sorted, and the same multiset checksum.
    out64 = work.to(torch.int64) & 0xFFFFFFFF
    is_sorted = bool((out64[1:] >= out64[:-1]).all().item())
    same_sum = int(out64.sum().item()) == int((src.to(torch.int64) & 0xFFFFFFFF).sum().item())
    del out64
    verified = is_sorted and same_sum
    log(f"[bench] sort: {ms_per_step:.3f} ms/step, {gkeys:.2f} Gkeys/s, "
        f"onesweep pass {pass_ms:.3f} ms ({pass_gbs:.0f} GB/s), verified={verified}")

    # ----------------------------------------------------------- CPU baseline
    cpu = None
    if not args.no_cpu:
        from oracle import cpu_oracle as O
        m = 1 << min(args.cpu_log2n, args.log2n)
        sample = src[:m].cpu().numpy().view(np.uint32)
        log(f"[bench] CPU baseline: oracle radix sort of the first 2^{int(np.log2(m))} keys")
        t0 = time.perf_counter()
        ref = O.radix_sort(sample)
        dt = time.perf_counter() - t0
        cpu = {"value": round(m / dt / 1e9, 5), "unit": "Gkeys/s", "cores": 1,
               "kind": "port",
               "sample": f"first 2^{int(np.log2(m))} keys of the workload, "
                         f"{dt:.1f} s, C restatement of the CPUAccelerator "
                         "path (16 virtual groups run in sequence, 2-bit "
                         "digits, 16 passes)",
               "host_cores": os.cpu_count()}
        # the same sample through the GPU path must agree bit for bit
        d = D.from_numpy(sample)
        capi.radix_sort_keys(d)
        torch.cuda.synchronize()
        verified = verified and bool(np.array_equal(d.numpy(), ref))
        del d, ref, sample

    result = {
        "metric": "radix_sort_u32_gkeys_per_s",
        "value": round(gkeys, 3),
        "unit": "Gkeys/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_statistic": "median",
        "mean_ms_per_step": round(mean_ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": f"RadixSort ascending, 2^{args.log2n} uint32 keys, "
                               "uniform over the full 32-bit range "
                               "(SplitMix64 seed 0x123456789ABCDEF0)",
                   "n": n, "passes_executed": passes,
                   "algorithmic_bytes_per_key": 4 * (2 * passes + 1)},
        "roofline": dict(roofline(pass_gbs, *measured_traffic(
                             "radix_sort_u32_uniform_2^28", args.log2n == 28)),
                         kernel="onesweep_pipelined_kernel<4, false>",
                         bytes_per_launch=pass_bytes,
                         avg_launch_ms=round(pass_ms, 4),
                         launches=pass_launches),
        "whole_sort": {"algorithmic_gbs": round(sort_gbs, 1),
                       "frac_of_hbm_peak": round(sort_gbs / HBM_PEAK_GBS, 4),
                       "kernel_avg_ms": kernel_ms,
                       "wall_s_timed_region": round(wall, 3)},
        "cpu_baseline": cpu,
        "verified": verified,
    }
    del src, work, keys, temp
    torch.cuda.empty_cache()

    if not args.no_extras:
        result["other_workloads"] = run_extras(args, torch, capi, datagen, timer, wrap)

    print(json.dumps(result), flush=True)


def run_extras(args, torch, capi, datagen, timer, wrap):
    """Scan, reduce, histogram, pairs and the skewed sorts at their baseline
    sizes; fewer steps than the headline."""
    D = capi.DeviceArray
    K = max(3, args.steps // 2)
    W = 2
    out = {}
    cpu_on = not args.no_cpu
    if cpu_on:
        from oracle import cpu_oracle as O

    def timed(name, prepare, fn, algo_bytes, kernel, kernel_bytes=None):
        ms, _ = timer.run(prepare, fn, K, W)
        capi.profile_enable(True)
        timer.run(prepare, fn, K, 0)
        launches, k_ms = kernel_stats(capi, kernel)
        capi.profile_enable(False)
        t = float(np.median(ms))
        kb = kernel_bytes if kernel_bytes is not None else algo_bytes
        k_gbs = kb / (k_ms * 1e-3) / 1e9 if k_ms else 0.0
        entry = {"ms_per_step": round(t, 4),
                 "mean_ms_per_step": round(float(np.mean(ms)), 4),
                 "algorithmic_gbs": round(algo_bytes / (t * 1e-3) / 1e9, 1),
                 "frac_of_hbm_peak": round(algo_bytes / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                 "roofline": dict(roofline(k_gbs, *measured_traffic(name, args.log2n == 28)),
                                  kernel=kernel, avg_launch_ms=round(k_ms, 4))}
        out[name] = entry
        log(f"[bench] {name}: {t:.3f} ms/step, {entry['algorithmic_gbs']:.0f} GB/s "
            f"({100 * entry['frac_of_hbm_peak']:.1f}% of peak)")
        return entry

    nothing = lambda: None
    n28 = 1 << min(28, args.log2n)

    # Exclusive Add scan of 2^28 int32 in [0, 15]
    x = datagen.small_ints_i32_torch(n28)
    y = torch.empty_like(x)
    d_in, d_out = wrap(x, np.int32), wrap(y, np.int32)
    temp = capi.temp_buffer(capi.scan_temp_bytes(n28, np.int32))
    e = timed("scan_exclusive_add_i32_2^28", nothing,
              lambda: capi.scan(d_in, d_out, temp, kind=capi.SCAN_EXCLUSIVE),
              2.0 * n28 * 4, "scan")
    expect = torch.cumsum(x, 0, dtype=torch.int64) - x
    e["verified"] = bool((y.to(torch.int64) == expect).all().item())
    del expect
    if cpu_on:
        m = 1 << 26
        s = x[:m].cpu().numpy()
        t0 = time.perf_counter(); O.scan(s, inclusive=False); dt = time.perf_counter() - t0
        e["cpu_baseline"] = {"value": round(2.0 * m * 4 / dt / 1e9, 3), "unit": "GB/s",
                             "cores": 1, "kind": "port", "sample": f"2^26 elements, {dt:.2f} s"}
    del x, y, d_in, d_out, temp

    # Add reduce of 2^28 float32 N(0,1)
    f = datagen.normal_f32_torch(n28)
    d_in, d_out = wrap(f, np.float32), D.zeros(1, np.float32)
    temp = capi.temp_buffer(capi.reduce_temp_bytes(n28, np.float32))
    e = timed("reduce_add_f32_2^28", nothing, lambda: capi.reduce(d_in, d_out, temp),
              n28 * 4.0, "reduce_partials")
    exact = float(f.to(torch.float64).sum().item())
    got = float(d_out.numpy()[0])
    e["result"], e["float64_sum"] = got, exact
    e["verified"] = abs(got - exact) <= 1e-5 * abs(exact) + abs(exact) * 2.0 ** -24
    if cpu_on:
        m = 1 << 26
        s = f[:m].cpu().numpy()
        t0 = time.perf_counter(); O.reduce(s); dt = time.perf_counter() - t0
        e["cpu_baseline"] = {"value": round(m * 4.0 / dt / 1e9, 3), "unit": "GB/s",
                             "cores": 1, "kind": "port", "sample": f"2^26 elements, {dt:.2f} s"}
    del f, d_in, d_out, temp

    # Histogram of 2^30 uint8 samples into 256 bins
    n30 = 1 << min(30, args.log2n + 2)
    b = datagen.bytes_u8_torch(n30)
    d_in, bins, ov = wrap(b, np.uint8), D.zeros(256, np.int32), D.zeros(1, np.int32)
    e = timed("histogram_u8_256bins_2^30", lambda: bins.bytes.zero_(),
              lambda: capi.histogram(d_in, bins, ov), float(n30), "histogram")
    expect = torch.bincount(b.to(torch.int64) if n30 <= (1 << 28) else b[: 1 << 28].to(torch.int64), minlength=256)
    if n30 > (1 << 28):
        for c in range(1, n30 >> 28):
            expect += torch.bincount(b[c << 28:(c + 1) << 28].to(torch.int64), minlength=256)
    e["verified"] = bool(np.array_equal(bins.numpy().astype(np.int64), expect.cpu().numpy()))
    if cpu_on:
        m = 1 << 28
        s = b[:m].cpu().numpy()
        t0 = time.perf_counter(); O.histogram(s, np.zeros(256, dtype=np.int32)); dt = time.perf_counter() - t0
        e["cpu_baseline"] = {"value": round(m / dt / 1e9, 3), "unit": "GB/s", "cores": 1,
                             "kind": "port", "sample": f"2^28 samples, {dt:.2f} s"}
    del b, d_in, expect

    # 4096-bin histogram of 2^28 int32 keys from a mixture of 8 Gaussians
    g = datagen.gaussian_mixture_i32_torch(n28)
    d_in, bins = wrap(g, np.int32), D.zeros(4096, np.int32)
    e = timed("histogram_i32_4096bins_2^28", lambda: bins.bytes.zero_(),
              lambda: capi.histogram(d_in, bins, ov), n28 * 4.0, "histogram")
    expect = torch.bincount(g.to(torch.int64), minlength=4096)
    e["verified"] = bool(np.array_equal(bins.numpy().astype(np.int64), expect.cpu().numpy()))
    if cpu_on:
        m = 1 << min(28, args.log2n)
        s = g[:m].cpu().numpy()
        t0 = time.perf_counter(); O.histogram(s, np.zeros(4096, dtype=np.int32)); dt = time.perf_counter() - t0
        e["cpu_baseline"] = {"value": round(m * 4.0 / dt / 1e9, 3), "unit": "GB/s", "cores": 1,
                             "kind": "port", "sample": f"2^{int(np.log2(m))} keys, {dt:.2f} s"}
    del g, d_in, expect

    # RadixSortPairs of 2^27 uint64 keys with uint32 index payload
    n27 = 1 << min(27, args.log2n)
    k64 = datagen.splitmix64_torch(n27)
    wk, wv = torch.empty_like(k64), torch.empty(n27, dtype=torch.int32, device="cuda:0")
    dk, dv = wrap(wk, np.uint64), wrap(wv, np.uint32)
    temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n27, np.uint64, 4))
    e = timed("radix_sort_pairs_u64_u32_2^27", lambda: wk.copy_(k64),
              lambda: capi.radix_sort_pairs(dk, dv, temp, values_from_index=True),
              n27 * (8.0 * 17 + 4.0 * 16), "sort_onesweep", n27 * 2.0 * 12)
    e["gpairs_per_s"] = round(n27 / (e["ms_per_step"] * 1e-3) / 1e9, 3)
    # stability + permutation: keys[values] reproduces the output, keys sorted
    # (unsigned order = signed order after flipping the sign bit), ties by index
    flip = wk ^ (-(1 << 63))
    ok_sorted = bool((flip[1:] >= flip[:-1]).all().item())
    ok_perm = bool((k64[wv.to(torch.int64)] == wk).all().item())
    ties = wk[1:] == wk[:-1]
    ok_stable = bool((wv[1:][ties] > wv[:-1][ties]).all().item())
    e["verified"] = ok_sorted and ok_perm and ok_stable
    if cpu_on:
        m = 1 << min(23, args.log2n)
        sk = k64[:m].cpu().numpy().view(np.uint64)
        t0 = time.perf_counter()
        rk, rv = O.radix_sort_pairs(sk, np.arange(m, dtype=np.uint32))
        dt = time.perf_counter() - t0
        e["cpu_baseline"] = {"value": round(m / dt / 1e9, 5), "unit": "Gpairs/s", "cores": 1,
                             "kind": "port",
                             "sample": f"first 2^{int(np.log2(m))} pairs, {dt:.1f} s (32 passes of "
                                       "2 bits over 16-byte key/value records)"}
        # the same sample through the GPU path must agree bit for bit
        gk, gv = D.from_numpy(sk), D.zeros(m, np.uint32)
        capi.radix_sort_pairs(gk, gv, values_from_index=True)
        torch.cuda.synchronize()
        e["verified"] = e["verified"] and bool(np.array_equal(gk.numpy(), rk)) and \
            bool(np.array_equal(gv.numpy(), rv))
        del sk, rk, rv, gk, gv
    del k64, wk, wv, dk, dv, temp, flip

    # Sizes between one tile and the headline: 2^20 (the configuration the
    # reference's CPUAccelerator can run: compared bit for bit with the oracle
    # at full size unless the CPU leg is off), 2^22 and 2^24.  At these sizes
    # the launches count: the entry says how many kernels one sort launches.
    for log2m in (20, 22, 24):
        m = 1 << log2m
        part = datagen.uniform_u32_torch(m)
        wk = torch.empty_like(part)
        kv = wrap(wk, np.uint32)
        tp = capi.temp_buffer(capi.radix_sort_temp_bytes(m, np.uint32))
        ms, _ = timer.run(lambda: wk.copy_(part), lambda: capi.radix_sort_keys(kv, tp), K, W)
        capi.profile_enable(True)
        timer.run(lambda: wk.copy_(part), lambda: capi.radix_sort_keys(kv, tp), 1, 0)
        launches = sum(kernel_stats(capi, k)[0] for k in
                       ("zero_words", "sort_histogram", "sort_plan", "sort_onesweep",
                        "sort_finish", "sort_small"))
        capi.profile_enable(False)
        t = float(np.median(ms))
        if cpu_on:
            host = part.cpu().numpy().view(np.uint32)
            t0 = time.perf_counter(); ref = O.radix_sort(host); dt = time.perf_counter() - t0
            ok = bool(np.array_equal(wk.cpu().numpy().view(np.uint32), ref))
            del host, ref
        else:  # without the CPU leg: against the GPU's own sort of the same keys
            ref64 = torch.sort(part.to(torch.int64) & 0xFFFFFFFF)[0]
            ok = bool(((wk.to(torch.int64) & 0xFFFFFFFF) == ref64).all().item())
            del ref64
        passes, _ = capi.radix_sort_passes(tp, m, np.uint32)
        algo = m * 4.0 * (2 * passes + 1)
        out[f"radix_sort_u32_2^{log2m}"] = {
            "ms_per_step": round(t, 4), "gkeys_per_s": round(m / (t * 1e-3) / 1e9, 2),
            "passes_executed": passes, "kernel_launches": launches,
            "algorithmic_gbs": round(algo / (t * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(algo / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "verified": ok}
        if cpu_on:
            out[f"radix_sort_u32_2^{log2m}"]["cpu_baseline"] = {
                "value": round(m / dt / 1e9, 5), "unit": "Gkeys/s", "cores": 1,
                "kind": "port", "sample": f"all 2^{log2m} keys, {dt:.1f} s"}
        log(f"[bench] radix_sort_u32_2^{log2m}: {t:.4f} ms/step, "
            f"{m / (t * 1e-3) / 1e9:.1f} Gkeys/s, {launches} launches, verified={ok}")
        del part, wk, kv, tp

    # Skewed sorts: Zipf(1.1) over 2^16 values, and all keys equal
    for name, src in (("radix_sort_u32_zipf_2^28", datagen.zipf_u32_torch(n28)),
                      ("radix_sort_u32_all_equal_2^28",
                       torch.full((n28,), -559038737, dtype=torch.int32, device="cuda:0"))):
        work = torch.empty_like(src)
        keys = wrap(work, np.uint32)
        temp = capi.temp_buffer(capi.radix_sort_temp_bytes(n28, np.uint32))
        ms, _ = timer.run(lambda: work.copy_(src), lambda: capi.radix_sort_keys(keys, temp), K, W)
        capi.profile_enable(True)
        timer.run(lambda: work.copy_(src), lambda: capi.radix_sort_keys(keys, temp), 1, 0)
        capi.profile_enable(False)
        t = float(np.median(ms))
        o64 = work.to(torch.int64) & 0xFFFFFFFF
        ok = bool((o64[1:] >= o64[:-1]).all().item()) and \
            int(o64.sum().item()) == int((src.to(torch.int64) & 0xFFFFFFFF).sum().item())
        passes, _ = capi.radix_sort_passes(temp, n28, np.uint32)   # read from the sort's plan
        algo = n28 * 4.0 * (2 * passes + 1)
        out[name] = {"ms_per_step": round(t, 4),
                     "gkeys_per_s": round(n28 / (t * 1e-3) / 1e9, 2),
                     "passes_executed": passes,
                     "algorithmic_gbs": round(algo / (t * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(algo / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "verified": ok}
        if cpu_on:
            m = 1 << min(25, args.log2n)
            sample = src[:m].cpu().numpy().view(np.uint32)
            t0 = time.perf_counter(); ref = O.radix_sort(sample); dt = time.perf_counter() - t0
            out[name]["cpu_baseline"] = {
                "value": round(m / dt / 1e9, 5), "unit": "Gkeys/s", "cores": 1, "kind": "port",
                "sample": f"first 2^{int(np.log2(m))} keys, {dt:.1f} s (the CPU path runs all 16 "
                          "passes whatever the keys)"}
            dsample = D.from_numpy(sample)
            capi.radix_sort_keys(dsample)
            torch.cuda.synchronize()
            out[name]["verified"] = ok and bool(np.array_equal(dsample.numpy(), ref))
            del sample, ref, dsample
        log(f"[bench] {name}: {t:.3f} ms/step, {out[name]['gkeys_per_s']} Gkeys/s")
        del work, keys, temp, o64, src

    # The neighbours of sort and scan in user pipelines.
    # Unique on sorted Zipf keys (the sort -> unique pipeline): reads n keys,
    # writes the kept ones.
    src = torch.sort(datagen.zipf_u32_torch(n28).to(torch.int64) & 0xFFFFFFFF)[0].to(torch.int32)
    work = torch.empty_like(src)
    d, count = wrap(work, np.uint32), D.zeros(1, np.int64)
    temp = capi.temp_buffer(capi.unique_temp_bytes(n28, np.uint32))
    distinct = int(torch.unique_consecutive(src).numel())
    e = timed("unique_u32_sorted_zipf_2^28", lambda: work.copy_(src),
              lambda: capi.unique(d, count, temp), 4.0 * (n28 + distinct), "unique")
    kept = int(count.numpy()[0])
    e["kept"] = kept
    e["verified"] = kept == distinct and bool(
        (work[:kept] == torch.unique_consecutive(src)).all().item())
    # all-distinct input: every element is written back
    seq = torch.arange(n28, dtype=torch.int32, device="cuda:0")
    e = timed("unique_i32_all_distinct_2^28", lambda: work.copy_(seq),
              lambda: capi.unique(d, count, temp), 8.0 * n28, "unique")
    e["verified"] = int(count.numpy()[0]) == n28 and bool((work == seq).all().item())
    del src, seq, temp

    # Sequence (iota) and Initialize (fill) of 2^28 int32: n * 4 bytes written.
    d = wrap(work, np.int32)
    e = timed("sequence_i32_2^28", nothing, lambda: capi.sequence(d), 4.0 * n28, "sequence")
    e["verified"] = bool((work == torch.arange(n28, dtype=torch.int32, device="cuda:0")).all().item())
    e = timed("initialize_i32_2^28", nothing, lambda: capi.initialize(d, 7), 4.0 * n28,
              "initialize")
    e["verified"] = bool((work == 7).all().item())
    # Reorder by a random permutation: a gather, n * (4 + 4 + 4) bytes.
    perm = torch.randperm(n28, device="cuda:0", generator=torch.Generator("cuda:0").manual_seed(1)).to(torch.int32)
    source = datagen.uniform_u32_torch(n28)
    e = timed("reorder_u32_random_permutation_2^28", nothing,
              lambda: capi.reorder(wrap(source, np.uint32), d, wrap(perm, np.int32)),
              12.0 * n28, "reorder")
    e["verified"] = bool((work == source[perm.to(torch.int64)]).all().item())
    # Transform: i32 -> -i32 (n * 8 bytes) and the widening i32 -> i64 (n * 12 bytes).
    d_src = wrap(source, np.int32)
    e = timed("transform_negate_i32_2^28", nothing,
              lambda: capi.transform(d_src, d, capi.TRANSFORM_NEGATE), 8.0 * n28, "transform")
    e["verified"] = bool((work == -source).all().item())
    wide = torch.empty(n28, dtype=torch.int64, device="cuda:0")
    e = timed("transform_i32_to_i64_2^28", nothing,
              lambda: capi.transform(d_src, wrap(wide, np.int64)), 12.0 * n28, "transform")
    e["verified"] = bool((wide == source.to(torch.int64)).all().item())
    del work, perm, source, wide
    return out


if __name__ == "__main__":
    main()
