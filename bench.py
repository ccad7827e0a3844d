#!/usr/bin/env python3
"""Benchmark of the packed-int4 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one call of ``quadmul.gemm`` (the drop-in entry point) on operands already
resident in HBM.  Prints ONE JSON line:

* ``metric``/``value``/``roofline``: the headline workload, by default the largest
  single-GPU configuration of the contract (M=N=K=8192): every input is made first, the
  kernel runs untimed for ``--preheat-ms`` (``config.preheat_ms``: the power management
  settles on the kernel's own load), then W untimed calls, then exactly K calls between
  two ``torch.cuda.synchronize()`` (wall clock -> ``value``, ``ms_per_step``) with one HIP
  event per step recorded on the stream the kernels are launched on (first to last:
  average launch duration -> ``roofline.achieved``; median, min and max beside it);
* ``targets``: every other configuration of the contract (1024^3, 4096^3, M in {1, 16, 64}
  at N=K=4096, the three M=2048 MLP shapes, 8000x8000x8064), each with its own
  ``roofline``.  These are timed the way the reference's harness times its kernel
  (test.py:60-107): launches captured into a HIP graph, replayed five times, the MEDIAN
  replay reported per launch.  HBM-bound shapes are reported with the launches rotating
  over copies of B that exceed the memory-side cache (B really comes from HBM), the
  figure on one cache-resident B beside it;
* ``mfma_issue_peak`` / ``launch_floor``: what the part itself sustains (a loop of the
  GEMM's MFMA instruction alone; an empty kernel and a read-only kernel per launch);
* ``cpu_baseline``: the CPU oracle (a restatement of the reference's ``cpu_gemm_int8``)
  timed on this box's host cores on a bounded sample of the headline workload and on
  configuration [0] (1024^3) in full, which also checks the GPU result bit for bit.
"""
from __future__ import annotations

import argparse
import glob
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5033.2   # dense int8 MFMA: 256 CU x 8192 op/clk/CU x 2.4 GHz
HBM_PEAK_GBS = 8000.0
SEED_BASE = 0x51AD0000

# name: (row of the contract's configuration table = seed offset, M, N, K, bound)
WORKLOADS = {
    "square1024": (0, 1024, 1024, 1024, "mfma"),      # configuration [0], the CPU path's own case
    "square4096": (1, 4096, 4096, 4096, "mfma"),      # [1]
    "skinny1": (2, 1, 4096, 4096, "hbm"),             # [2]
    "skinny16": (3, 16, 4096, 4096, "hbm"),
    "skinny64": (4, 64, 4096, 4096, "hbm"),
    "mlp_up": (5, 2048, 11008, 4096, "mfma"),         # [3]
    "mlp_down": (6, 2048, 4096, 11008, "mfma"),
    "qkv": (7, 2048, 12288, 4096, "mfma"),
    "square8192": (8, 8192, 8192, 8192, "mfma"),      # [4], the headline
    "tail8000": (9, 8000, 8000, 8064, "mfma"),
    # the skinny target's kernel at a size where the launch no longer dominates (an extra, not a row of the contract)
    "skinny16_wide": (10, 16, 28672, 4096, "hbm"),
}
HEADLINE = "square8192"


def algorithmic_bytes(m, n, k):
    return m * k // 2 + n * k // 2 + 4 * m * n


def make_packed(m, n, k, seed):
    """Seeded int4 values on the inclusive range [-8, 7], packed low nibble = even k."""
    import numpy as np
    import torch

    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=g)
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=g)

    def pack(v):
        u = v.numpy().view(np.uint8)
        return torch.from_numpy(np.ascontiguousarray((u[:, 0::2] & 0x0F) | ((u[:, 1::2] & 0x0F) << 4)).view(np.int8))

    return pack(a), pack(b)


def time_steps(fn, steps, warmup, preheat_ms=0.0):
    """Exactly `steps` calls after `warmup` untimed ones: wall ms per step, and from one HIP
    event per step on the launch stream the mean / median / min / max step in ms.

    `preheat_ms` > 0: before the warm-ups the same kernel runs back to back for at least that
    long, untimed.  A burst of launches that follows an idle GPU starts with a power-management
    transient (the first four launches of 8192^3 at 0.36 ms, launches 6..12 at 0.43-0.46 ms,
    then a slow return to the sustained 0.33 ms over about 80 launches = 30 ms, whatever the
    length of the idle gap); the timing method this follows (kernel.cu:472-497: 10 warm-ups,
    100 trials) averages over it, a run of 5 + 20 launches does not."""
    import torch

    pre = {"preheat_ms": 0.0, "preheat_launches": 0}
    if preheat_ms > 0:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        n = max(1, int(preheat_ms / max(e0.elapsed_time(e1), 1e-3)) + 1)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        pre_events = (e0, e1, n)
    for _ in range(warmup):
        fn()
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    evs[0].record()
    for i in range(steps):
        fn()
        evs[i + 1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per = [evs[i].elapsed_time(evs[i + 1]) for i in range(steps)]
    if preheat_ms > 0:
        pre = {"preheat_ms": round(pre_events[0].elapsed_time(pre_events[1]), 1), "preheat_launches": pre_events[2]}
    stats = {"mean": evs[0].elapsed_time(evs[steps]) / steps, "median": statistics.median(per), "min": min(per), "max": max(per)}
    return wall, stats, pre


def time_graph(fn, launches=200, replays=5):
    """ms per launch with the launches captured into one HIP graph (the reference's own
    timing method, test.py:78-91): removes the host's per-call cost for short kernels.
    One untimed replay, then `replays` timed ones: (median, min, max)."""
    import torch

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()
        with torch.cuda.graph(g, stream=side):
            for _ in range(launches):
                fn()
    torch.cuda.current_stream().wait_stream(side)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ts = []
    for _ in range(replays):
        e0.record()
        g.replay()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) / launches)
    return statistics.median(ts), min(ts), max(ts)


# Bytes moved per launch past the L2s come from the committed rocprofv3 summaries, not from
# this run: two --pmc runs of `bench.py --workload W --launches-only 20` (FETCH_SIZE, then
# WRITE_SIZE; KiB per dispatch, each scaled by what the same counter reads for a 256 MiB
# device-to-device copy) per workload, summarised in profiles/<kernel>_<configuration>__<W>.md.
# A summary is used only while the configuration it profiled is still the one the library
# chooses for that shape; a retuned table row leaves `traffic` null until it is profiled again.
_TITLE = re.compile(r"^# (\S+?)_kernel, configuration (\S+?),(?: [^\n]*?)? on (\S+) \(M=(\d+) N=(\d+) K=(\d+)\)")
_TOTAL = re.compile(r"^\| total \| \| (\d+) \|", re.M)


def profile_summaries(root=None):
    """{workload: {"path", "kernel", "config", "shape", "traffic"}} for every profiles/*__<workload>.md
    with a traffic table."""
    out = {}
    for path in sorted(glob.glob(os.path.join(root or ROOT, "profiles", "*__*.md"))):
        with open(path) as f:
            text = f.read()
        title = _TITLE.match(text)
        total = _TOTAL.search(text)
        if not title or not total:
            continue
        out[title.group(3)] = {"path": "profiles/" + os.path.basename(path), "kernel": title.group(1), "config": title.group(2),
                               "shape": tuple(int(title.group(i)) for i in (4, 5, 6)), "traffic": int(total.group(1))}
    return out


def profile_total(workload):
    """The traffic total of profiles/*__<workload>.md whatever its title says (summaries of the
    kernels either side of the GEMM), or None."""
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", f"*__{workload}.md"))):
        with open(path) as f:
            total = _TOTAL.search(f.read())
        if total:
            return int(total.group(1))
    return None


def profiled_traffic(name, m, n, k, config):
    """(bytes per launch, where from) for workload `name` running configuration `config`."""
    prof = profile_summaries().get(name)
    if prof is None:
        return None, "no rocprofv3 summary of this workload under profiles/"
    if prof["shape"] != (m, n, k) or prof["config"] != config:
        return None, f"{prof['path']} profiled {prof['config']}, the library now chooses {config}: not used"
    return prof["traffic"], f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiled offline ({prof['path']})"


def roofline_of(m, n, k, bound, ms, issue_peak_tops=None, name=None, config=None):
    ops = 2.0 * m * n * k
    traffic, source = profiled_traffic(name, m, n, k, config) if name else (None, None)
    if bound == "mfma":
        achieved, peak, unit = ops / ms / 1e9, INT8_PEAK_TOPS, "TOP/s"
    else:
        achieved, peak, unit = algorithmic_bytes(m, n, k) / ms / 1e6, HBM_PEAK_GBS, "GB/s"
    r = {"bound": bound, "achieved": round(achieved, 1), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
         "traffic": traffic, "traffic_source": source, "algorithmic_bytes": algorithmic_bytes(m, n, k), "launch_us": round(ms * 1e3, 3)}
    if bound == "mfma" and issue_peak_tops:
        r["frac_of_measured_issue_peak"] = round(achieved / issue_peak_tops, 4)
    return r


def check_rows(ap, bp, c_d, m, count=8):
    """`count` evenly spaced rows of the GPU result against the CPU oracle, bit for bit."""
    import numpy as np

    import oracle

    rows = np.unique(np.linspace(0, m - 1, min(count, m)).astype(np.int32))
    want = oracle.gemm_i4_rows(ap.numpy(), bp.numpy(), rows, threads=0)
    return bool((c_d[rows.tolist()].cpu().numpy() == want).all()), int(rows.size)


def workload_text(name):
    row, m, n, k, _ = WORKLOADS[name]
    return (f"{name}: M={m} N={n} K={k}, signed int4 packed 2/byte along K (low nibble = even k), "
            f"C=A.B^T int32, uniform [-8,7] seed {hex(SEED_BASE + row)}")


def run_target(name, issue_peak_tops):
    """One configuration of the contract as a `targets` entry: graph-timed, median of the replays."""
    import torch

    import quadmul            # the drop-in extension module
    import quadmul_amd as qm  # config introspection only

    row, m, n, k, bound = WORKLOADS[name]
    ap, bp = make_packed(m, n, k, SEED_BASE + row)
    dev = torch.device("cuda:0")
    a_d, b_d = ap.to(dev), bp.to(dev)
    c_d = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    exact, nrows = check_rows(ap, bp, c_d, m)
    # about 50 ms of launches per replay
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    est_ms = max((time.perf_counter() - t0) * 1e3 * 0.5, 2e-3)
    launches = int(min(2000, max(20, 50.0 / est_ms)))
    med, lo, hi = time_graph(fn, launches=launches)
    config = qm.config_name(qm.select_config(m, n, k) & 0xFFFF)
    out = {
        "workload": workload_text(name), "m": m, "n": n, "k": k,
        "kernel": config,
        "timing": f"HIP graph of {launches} launches, median of 5 replays",
        "ms_per_launch": round(med, 5), "ms_per_launch_min_max": [round(lo, 5), round(hi, 5)],
        "tops": round(2.0 * m * n * k / med / 1e9, 2),
        "gbs_algorithmic": round(algorithmic_bytes(m, n, k) / med / 1e6, 1),
        "rows_checked_against_cpu_oracle": nrows, "rows_bit_exact": exact,
    }
    if bound == "hbm":
        # Launched again and again on the same B, the kernel reads B out of the L2s and the
        # 256 MiB memory-side cache, not HBM.  For the HBM roofline the launches of the graph
        # rotate over enough copies of B (each with a C of its own) to exceed that cache.
        fn_rot, ncopies, cs = rotating_call(a_d, b_d, c_d, m, n, k)
        rot, rlo, rhi = time_graph(fn_rot, launches=5 * ncopies)
        for c_i in cs[1:]:
            assert torch.equal(c_i, c_d)
        del fn_rot, cs
        out["ms_per_launch_rotating_b"] = round(rot, 5)
        out["ms_per_launch_rotating_b_min_max"] = [round(rlo, 5), round(rhi, 5)]
        out["roofline"] = roofline_of(m, n, k, bound, rot, name=name + "_rotating_b", config=config)
        out["roofline"]["note"] = (f"launches rotate over {ncopies} copies of B (> 256 MiB memory-side cache): B comes from HBM; "
                                   f"graph of {5 * ncopies} launches, median of 5 replays")
        out["roofline_b_cache_resident"] = roofline_of(m, n, k, bound, med, name=name, config=config)
    else:
        out["roofline"] = roofline_of(m, n, k, bound, med, issue_peak_tops, name=name, config=config)
    return out, (ap, bp, a_d, b_d, c_d)


def extras_4096(a_d, b_d, c_d):
    """The callers either side of the GEMM at 4096^3: the fused dequantising epilogue (fp16
    out) and quantise + pack of a [4096, 4096] fp16 activation matrix."""
    import torch

    import quadmul
    import quadmul_amd as qm

    m = n = k = 4096
    dev = a_d.device
    rs = torch.rand(m, device=dev) * 0.02 + 1e-3
    cs = torch.rand(n, device=dev) * 0.05 + 1e-4
    d_d = torch.empty((m, n), dtype=torch.float16, device=dev)
    fn_s = lambda: quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
    fn_s()
    torch.cuda.synchronize()
    s_ms, _, _ = time_graph(fn_s)
    want = ((c_d.to(torch.float32) * rs[:, None]) * cs[None, :]).to(torch.float16)
    assert torch.equal(d_d.view(torch.int16), want.view(torch.int16)), "scaled output differs from its definition"
    x = torch.randn((m, k), device=dev).to(torch.float16)
    q_ms, _, _ = time_graph(lambda: quadmul.quantize_pack(x), launches=50)
    q_bytes = m * k * 2 + m * k // 2 + 4 * m
    return {
        "scaled_fp16_output": {"entry_point": "quadmul.gemm_scaled(a, b, d, m, n, k, row_scale, col_scale)",
                               "ms_per_launch": round(s_ms, 5), "tops": round(2.0 * m * n * k / s_ms / 1e9, 1),
                               "frac_of_int8_peak": round(2.0 * m * n * k / s_ms / 1e9 / INT8_PEAK_TOPS, 4),
                               "algorithmic_bytes": m * k // 2 + n * k // 2 + 2 * m * n + 4 * (m + n),
                               "traffic": profiled_traffic("square4096_scaled_f16", m, n, k, qm.config_name(qm.select_config_ex(m, n, k, scaled=True) & 0xFFFF))[0],
                               "checked": "every element against torch's float32 arithmetic on the int32 result"},
        "quantize_pack_fp16": {"entry_point": "quadmul.quantize_pack(x)", "rows": m, "k": k, "ms_per_launch": round(q_ms, 5),
                               "algorithmic_bytes": q_bytes,
                               "roofline": {"bound": "hbm", "achieved": round(q_bytes / q_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                            "frac": round(q_bytes / q_ms / 1e6 / HBM_PEAK_GBS, 4),
                                            "traffic": profile_total("quantize4096_f16")}},
    }


def cpu_baseline(ap, bp, c_gpu, m, n, k):
    """The CPU oracle (a restatement of the reference's cpu_gemm_int8) on a bounded sample
    of the headline workload -- a block of rows of A against all of B -- and on configuration
    [0] (1024^3) in full; also checks the GPU result for those rows bit-exactly."""
    import numpy as np

    import oracle

    threads = oracle.max_threads()
    # budgets in MACs: about 10 s on all cores, about 10 s on one core (measured rates:
    # ~1.5e10 MAC/s per core)
    rows_mt = min(m, max(16, int(1.5e10 * 10 * min(threads, 8) / (n * k))))
    rows_1t = min(m, max(4, int(1.5e10 * 10 / (n * k))))
    sel_mt = np.unique(np.linspace(0, m - 1, rows_mt).astype(np.int32))
    rows_mt = int(sel_mt.size)
    t0 = time.perf_counter()
    c_mt = oracle.gemm_i4_rows(ap.numpy(), bp.numpy(), sel_mt, threads=0)
    t_mt = time.perf_counter() - t0
    sel_1t = sel_mt[:rows_1t]
    rows_1t = int(sel_1t.size)
    t0 = time.perf_counter()
    c_1t = oracle.gemm_i4_rows(ap.numpy(), bp.numpy(), sel_1t, threads=1)
    t_1t = time.perf_counter() - t0
    got = c_gpu.cpu().numpy()
    exact = bool((got[sel_mt] == c_mt).all() and (got[sel_1t] == c_1t).all())
    tops_mt = 2.0 * rows_mt * n * k / t_mt / 1e12
    tops_1t = 2.0 * rows_1t * n * k / t_1t / 1e12
    # configuration [0]: M=N=K=1024 in full, unpack first as the reference's main does
    # (kernel.cu:447-448,505); best of three, the run being short
    a0, b0 = make_packed(1024, 1024, 1024, SEED_BASE + 0)
    t1 = min(_timed(lambda: oracle.gemm_i4(a0.numpy(), b0.numpy(), threads=1)) for _ in range(3))
    tm = min(_timed(lambda: oracle.gemm_i4(a0.numpy(), b0.numpy(), threads=0)) for _ in range(3))
    return {
        "value": round(tops_mt, 5), "unit": "TOPS", "cores": threads, "kind": "port",
        "sample": f"{rows_mt} of {m} rows of A (evenly spaced) x all {n} rows of B, K={k}; unpack + triple loop "
                  f"as kernel.cu:291-306,389-408, OpenMP over rows, {t_mt:.2f} s",
        "single_thread": {"value": round(tops_1t, 5), "unit": "TOPS", "cores": 1,
                          "sample": f"{rows_1t} rows, the reference's loop nest unchanged, {t_1t:.2f} s"},
        "config0_1024cubed": {"single_thread_ms": round(t1 * 1e3, 2), "single_thread_gops": round(2.0 * 1024 ** 3 / t1 / 1e9, 2),
                              "all_cores_ms": round(tm * 1e3, 2), "all_cores_gops": round(2.0 * 1024 ** 3 / tm / 1e9, 2), "cores": threads,
                              "sample": "M=N=K=1024 in full, unpack + triple loop, best of 3"},
        "gpu_rows_bit_exact": exact,
    }


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def rotating_call(a_d, b_d, c_d, m, n, k):
    """A call that rotates over enough copies of B (each with a C of its own) to exceed the
    256 MiB memory-side cache, so that B comes from HBM: (callable, copies, the outputs)."""
    import torch

    import quadmul

    ncopies = max(2, -(-(320 << 20) // max(1, b_d.numel())))
    bs = [b_d] + [b_d.clone() for _ in range(ncopies - 1)]
    cs = [c_d] + [torch.empty_like(c_d) for _ in range(ncopies - 1)]
    turn = [0]

    def fn_rot():
        i = turn[0] % ncopies
        turn[0] += 1
        quadmul.gemm(a_d, bs[i], cs[i], m, n, k)

    return fn_rot, ncopies, cs


def launches_only(a):
    """Profiling aid: just N launches of one workload (after one warm-up), nothing else."""
    import torch

    import quadmul

    dev = "cuda:0"
    if a.workload == "quantize4096_f16":
        x = torch.randn((4096, 4096), device=dev).to(torch.float16)
        for _ in range(a.launches_only + 1):
            quadmul.quantize_pack(x)
    elif a.workload == "square4096_scaled_f16":
        row, m, n, k, _ = WORKLOADS["square4096"]
        apk, bpk = make_packed(m, n, k, SEED_BASE + row)
        a_d, b_d = apk.to(dev), bpk.to(dev)
        d_d = torch.empty((m, n), dtype=torch.float16, device=dev)
        rs, cs = torch.rand(m, device=dev) * 0.02 + 1e-3, torch.rand(n, device=dev) * 0.05 + 1e-4
        for _ in range(a.launches_only + 1):
            quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
    else:
        row, m, n, k, _ = WORKLOADS[a.workload]
        apk, bpk = make_packed(m, n, k, SEED_BASE + row)
        a_d, b_d = apk.to(dev), bpk.to(dev)
        c_d = torch.empty((m, n), dtype=torch.int32, device=dev)
        fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
        if a.rotate_b:
            fn, _, _ = rotating_call(a_d, b_d, c_d, m, n, k)
        for _ in range(a.launches_only + 1):
            fn()
    torch.cuda.synchronize()
    print(json.dumps({"launches_only": a.launches_only, "workload": a.workload, "rotate_b": bool(a.rotate_b)}))
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS) + ["square4096_scaled_f16", "quantize4096_f16"],
                    help="the workload of the JSON line's value; the last two names exist for --launches-only (profiling) only")
    ap.add_argument("--preheat-ms", type=float, default=400.0,
                    help="untimed back-to-back launches of the headline kernel for this long before the warm-ups, so that the "
                         "timed steps run at the sustained clock (0: none)")
    ap.add_argument("--no-targets", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-probes", action="store_true", help="skip the MFMA issue and launch floor probes")
    ap.add_argument("--launches-only", type=int, default=0, metavar="N",
                    help="profiling aid: just N launches of --workload (after one warm-up), nothing else")
    ap.add_argument("--graph-only", type=int, default=0, metavar="N",
                    help="profiling aid: one HIP graph of N launches of --workload, replayed six times, nothing else")
    ap.add_argument("--rotate-b", action="store_true",
                    help="with --launches-only / --graph-only: the launches rotate over copies of B that exceed the memory-side "
                         "cache, so that B comes from HBM")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="profiling aid: ten device-to-device copies of 256 MiB (a plain copy kernel of known "
                         "size, to scale the FETCH_SIZE / WRITE_SIZE counters)")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        print("bench.py: this hot path is a single-GPU kernel and every box here has one GPU; "
              "run with --gpus 1 (row blocks of A or of B shard with no exchange; a split of K needs one int32 all-reduce)", file=sys.stderr)
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the int4 GEMM)", file=sys.stderr)
        return 2

    if a.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(3)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read_per_copy": 256 << 20, "bytes_written_per_copy": 256 << 20, "copies": 10}}))
        return 0
    if a.launches_only:
        return launches_only(a)
    if a.workload not in WORKLOADS:
        print("bench.py: that workload name is for --launches-only", file=sys.stderr)
        return 2
    if a.graph_only:
        import quadmul

        row, m, n, k, _ = WORKLOADS[a.workload]
        apk, bpk = make_packed(m, n, k, SEED_BASE + row)
        a_d, b_d = apk.to("cuda:0"), bpk.to("cuda:0")
        c_d = torch.empty((m, n), dtype=torch.int32, device="cuda:0")
        fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
        if a.rotate_b:
            fn, _, _ = rotating_call(a_d, b_d, c_d, m, n, k)
        med, lo, hi = time_graph(fn, launches=a.graph_only)
        print(json.dumps({"graph_only": a.graph_only, "workload": a.workload, "rotate_b": bool(a.rotate_b), "ms_per_launch_median": round(med, 5),
                          "min_max": [round(lo, 5), round(hi, 5)]}))
        return 0

    import quadmul
    import quadmul_amd as qm

    # every input is made and moved to the GPU before anything is timed: nothing but kernels
    # runs between the probes and the timed steps
    row, m, n, k, bound = WORKLOADS[a.workload]
    apk, bpk = make_packed(m, n, k, SEED_BASE + row)
    dev = torch.device("cuda:0")
    a_d, b_d = apk.to(dev), bpk.to(dev)
    c_d = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
    fn()
    torch.cuda.synchronize()

    probes = {}
    issue_peak = None
    if not a.no_probes:
        from quadmul_amd import probe

        probes["mfma_issue_peak"] = probe.mfma_issue_peak()
        probes["launch_floor"] = probe.launch_floor()
        issue_peak = probes["mfma_issue_peak"]["tops"]

    # ---- the headline: exactly `steps` calls of quadmul.gemm after `warmup` untimed ones ----
    wall_ms, ev, pre = time_steps(fn, a.steps, a.warmup, a.preheat_ms)
    event_ms = ev["mean"]
    graph_med, graph_lo, graph_hi = time_graph(fn, launches=int(min(2000, max(20, 50.0 / max(event_ms, 2e-3)))))
    config = qm.config_name(qm.select_config(m, n, k) & 0xFFFF)
    line = {
        "metric": "int4 GEMM TOPS and % of int8 MFMA peak / % HBM BW, 1xMI355X",
        "value": round(2.0 * m * n * k / wall_ms / 1e9, 2), "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8 (s4 nibbles widened to 16*s4) x i8 -> i32 MFMA, exact",
        "data": "synthetic",
        "config": {"workload": workload_text(a.workload), "kernel": config,
                   "entry_point": "quadmul.gemm(a, b, c, m, n, k)",
                   # untimed launches of the same kernel before the warm-ups (see time_steps)
                   "preheat_ms": pre["preheat_ms"], "preheat_launches": pre["preheat_launches"],
                   "ms_per_step_events": round(event_ms, 5), "ms_per_step_events_median": round(ev["median"], 5),
                   "ms_per_step_events_min_max": [round(ev["min"], 5), round(ev["max"], 5)],
                   "ms_per_launch_graph_median": round(graph_med, 5), "ms_per_launch_graph_min_max": [round(graph_lo, 5), round(graph_hi, 5)]},
        # average launch duration over the timed steps, from the HIP events around them
        "roofline": roofline_of(m, n, k, bound, event_ms, issue_peak, name=a.workload, config=config),
    }
    line["roofline"]["duration_source"] = (f"one HIP event per step on the launch stream: first to last over the {a.steps} timed steps, average per launch "
                                           f"(after {pre['preheat_launches']} untimed launches = {pre['preheat_ms']} ms of the same kernel and {a.warmup} warm-ups)")
    line.update(probes)
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(apk, bpk, c_d, m, n, k)
    else:
        exact, nrows = check_rows(apk, bpk, c_d, m)
        line["config"]["rows_bit_exact"] = exact
    del apk, bpk, a_d, b_d, c_d
    torch.cuda.empty_cache()
    if not a.no_targets:
        targets = []
        for name in WORKLOADS:
            if name == a.workload:
                continue
            res, (tap, tbp, ta_d, tb_d, tc_d) = run_target(name, issue_peak)
            if name == "square4096":
                res.update(extras_4096(ta_d, tb_d, tc_d))
            targets.append(res)
            del tap, tbp, ta_d, tb_d, tc_d
            torch.cuda.empty_cache()
        line["targets"] = targets
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
