#!/usr/bin/env python3
"""Benchmark of the packed-int4 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one call of ``quadmul.gemm`` (the drop-in entry point) on operands already
resident in HBM.  Prints ONE JSON line:

* ``metric``/``value``/``roofline``: the headline workload, by default the largest
  single-GPU configuration of the contract (M=N=K=8192): W untimed calls, then exactly K
  calls between two ``torch.cuda.synchronize()`` (wall clock -> ``value``, ``ms_per_step``)
  and, inside them, between two HIP events recorded on the stream the kernels are
  launched on (average launch duration -> ``roofline.achieved``);
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
import json
import os
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


def time_steps(fn, steps, warmup):
    """(wall ms per step, event ms per step) over exactly `steps` calls."""
    import torch

    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, e0.elapsed_time(e1) / steps


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


# Bytes moved per launch past the L2s, profiled offline: two rocprofv3 --pmc runs of
# `bench.py --workload W --launches-only 20` (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch,
# each scaled by what the same counter reads for a 256 MiB device-to-device copy); the
# summaries are under profiles/.  Not measured in this run.
PROFILED_TRAFFIC = {(8192, 8192, 8192): 673454571, (8000, 8000, 8064): 768061246, (4096, 4096, 4096): 118719686, (2048, 11008, 4096): 192246061,
                    (2048, 4096, 11008): 124369042, (16, 28672, 4096): 60893081,
                    (1024, 1024, 1024): 7542887, (16, 4096, 4096): 8993197, (64, 4096, 4096): 10607970, (1, 4096, 4096): 8460539}
PROFILED_TRAFFIC_OTHER = {"scaled_fp16_4096^3": 85807335, "quantize_pack_fp16_4096x4096": 42113123}


def roofline_of(m, n, k, bound, ms, issue_peak_tops=None):
    ops = 2.0 * m * n * k
    if bound == "mfma":
        achieved = ops / ms / 1e9  # TOP/s
        r = {"bound": "mfma", "achieved": round(achieved, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
             "frac": round(achieved / INT8_PEAK_TOPS, 4), "traffic": PROFILED_TRAFFIC.get((m, n, k)),
             "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiled offline (profiles/)" if (m, n, k) in PROFILED_TRAFFIC else None,
             "algorithmic_bytes": algorithmic_bytes(m, n, k), "launch_us": round(ms * 1e3, 3)}
        if issue_peak_tops:
            r["frac_of_measured_issue_peak"] = round(achieved / issue_peak_tops, 4)
        return r
    achieved = algorithmic_bytes(m, n, k) / ms / 1e6  # GB/s
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": PROFILED_TRAFFIC.get((m, n, k)),
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiled offline (profiles/)" if (m, n, k) in PROFILED_TRAFFIC else None,
            "algorithmic_bytes": algorithmic_bytes(m, n, k), "launch_us": round(ms * 1e3, 3)}


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
    out = {
        "workload": workload_text(name), "m": m, "n": n, "k": k,
        "kernel": qm.config_name(qm.select_config(m, n, k) & 0xFFFF),
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
        ncopies = max(2, -(-(320 << 20) // max(1, bp.numel())))
        bs = [b_d] + [b_d.clone() for _ in range(ncopies - 1)]
        cs = [c_d] + [torch.empty_like(c_d) for _ in range(ncopies - 1)]
        turn = [0]

        def fn_rot():
            i = turn[0] % ncopies
            turn[0] += 1
            quadmul.gemm(a_d, bs[i], cs[i], m, n, k)

        rot, rlo, rhi = time_graph(fn_rot, launches=5 * ncopies)
        for c_i in cs[1:]:
            assert torch.equal(c_i, c_d)
        del bs, cs
        out["ms_per_launch_rotating_b"] = round(rot, 5)
        out["ms_per_launch_rotating_b_min_max"] = [round(rlo, 5), round(rhi, 5)]
        out["roofline"] = roofline_of(m, n, k, bound, rot)
        out["roofline"]["note"] = (f"launches rotate over {ncopies} copies of B (> 256 MiB memory-side cache): B comes from HBM; "
                                   f"graph of {5 * ncopies} launches, median of 5 replays")
        out["roofline_b_cache_resident"] = roofline_of(m, n, k, bound, med)
    else:
        out["roofline"] = roofline_of(m, n, k, bound, med, issue_peak_tops)
    return out, (ap, bp, a_d, b_d, c_d)


def extras_4096(a_d, b_d, c_d):
    """The callers either side of the GEMM at 4096^3: the fused dequantising epilogue (fp16
    out) and quantise + pack of a [4096, 4096] fp16 activation matrix."""
    import torch

    import quadmul

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
                               "traffic": PROFILED_TRAFFIC_OTHER["scaled_fp16_4096^3"],
                               "checked": "every element against torch's float32 arithmetic on the int32 result"},
        "quantize_pack_fp16": {"entry_point": "quadmul.quantize_pack(x)", "rows": m, "k": k, "ms_per_launch": round(q_ms, 5),
                               "algorithmic_bytes": q_bytes,
                               "roofline": {"bound": "hbm", "achieved": round(q_bytes / q_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                            "frac": round(q_bytes / q_ms / 1e6 / HBM_PEAK_GBS, 4),
                                            "traffic": PROFILED_TRAFFIC_OTHER["quantize_pack_fp16_4096x4096"]}},
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
        for _ in range(a.launches_only + 1):
            quadmul.gemm(a_d, b_d, c_d, m, n, k)
    torch.cuda.synchronize()
    print(json.dumps({"launches_only": a.launches_only, "workload": a.workload}))
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS) + ["square4096_scaled_f16", "quantize4096_f16"],
                    help="the workload of the JSON line's value; the last two names exist for --launches-only (profiling) only")
    ap.add_argument("--no-targets", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-probes", action="store_true", help="skip the MFMA issue and launch floor probes")
    ap.add_argument("--launches-only", type=int, default=0, metavar="N",
                    help="profiling aid: just N launches of --workload (after one warm-up), nothing else")
    ap.add_argument("--graph-only", type=int, default=0, metavar="N",
                    help="profiling aid: one HIP graph of N launches of --workload, replayed six times, nothing else")
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
        med, lo, hi = time_graph(lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k), launches=a.graph_only)
        print(json.dumps({"graph_only": a.graph_only, "workload": a.workload, "ms_per_launch_median": round(med, 5),
                          "min_max": [round(lo, 5), round(hi, 5)]}))
        return 0

    import quadmul
    import quadmul_amd as qm

    probes = {}
    issue_peak = None
    if not a.no_probes:
        from quadmul_amd import probe

        probes["mfma_issue_peak"] = probe.mfma_issue_peak()
        probes["launch_floor"] = probe.launch_floor()
        issue_peak = probes["mfma_issue_peak"]["tops"]

    # ---- the headline: exactly `steps` calls of quadmul.gemm after `warmup` untimed ones ----
    row, m, n, k, bound = WORKLOADS[a.workload]
    apk, bpk = make_packed(m, n, k, SEED_BASE + row)
    dev = torch.device("cuda:0")
    a_d, b_d = apk.to(dev), bpk.to(dev)
    c_d = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
    fn()
    torch.cuda.synchronize()
    wall_ms, event_ms = time_steps(fn, a.steps, a.warmup)
    graph_med, graph_lo, graph_hi = time_graph(fn, launches=int(min(2000, max(20, 50.0 / max(event_ms, 2e-3)))))
    line = {
        "metric": "int4 GEMM TOPS and % of int8 MFMA peak / % HBM BW, 1xMI355X",
        "value": round(2.0 * m * n * k / wall_ms / 1e9, 2), "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8 (s4 nibbles widened to 16*s4) x i8 -> i32 MFMA, exact",
        "data": "synthetic",
        "config": {"workload": workload_text(a.workload), "kernel": qm.config_name(qm.select_config(m, n, k) & 0xFFFF),
                   "entry_point": "quadmul.gemm(a, b, c, m, n, k)",
                   "ms_per_step_events": round(event_ms, 5),
                   "ms_per_launch_graph_median": round(graph_med, 5), "ms_per_launch_graph_min_max": [round(graph_lo, 5), round(graph_hi, 5)]},
        # average launch duration over the timed steps, from the HIP events around them
        "roofline": roofline_of(m, n, k, bound, event_ms, issue_peak),
    }
    line["roofline"]["duration_source"] = f"HIP events around the {a.steps} timed steps on the launch stream, average per launch"
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
