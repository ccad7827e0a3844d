#!/usr/bin/env python3
"""Benchmark of the packed-int4 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload square4096|square8192|skinny16|skinny1]

A step is one call of ``quadmul.gemm`` (the drop-in entry point) on operands already
resident in HBM.  Prints ONE JSON line: the throughput of the main workload
(``metric``/``value``), the roofline position of its kernel (``roofline``), the same
two figures for the other named target shapes (``targets``), and the CPU oracle timed
on this box's host cores on a bounded sample of the same workload (``cpu_baseline``).

Timing: W untimed calls, then exactly K calls between two ``torch.cuda.synchronize()``
(wall clock -> ``ms_per_step``) and, inside them, between two HIP events recorded on
the stream the kernels are launched on (-> ``roofline.achieved``).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5033.2   # dense int8 MFMA: 256 CU x 8192 op/clk/CU x 2.4 GHz
HBM_PEAK_GBS = 8000.0
SEED_BASE = 0x51AD0000

WORKLOADS = {
    # name: (config row, M, N, K, bound)
    "square4096": (1, 4096, 4096, 4096, "mfma"),
    "square8192": (8, 8192, 8192, 8192, "mfma"),
    "skinny16": (3, 16, 4096, 4096, "hbm"),
    "skinny1": (2, 1, 4096, 4096, "hbm"),
    # the skinny target's kernel at a size where the launch no longer dominates (an extra, not a BASELINE row)
    "skinny16_wide": (4, 16, 28672, 4096, "hbm"),
}


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
    timing method, test.py:78-91): removes the host's per-call cost for short kernels."""
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
    best = float("inf")
    for _ in range(replays):
        e0.record()
        g.replay()
        e1.record()
        e1.synchronize()
        best = min(best, e0.elapsed_time(e1) / launches)
    return best


# Bytes moved per launch past the L2s, from rocprofv3 counter runs of `bench.py --workload W
# --launches-only 20` (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads
# for a 256 MiB device-to-device copy; summaries under profiles/).  Not measured live.
MEASURED_TRAFFIC = {(4096, 4096, 4096): 118964029, (8192, 8192, 8192): 677540868, (16, 4096, 4096): 8956310, (1, 4096, 4096): 8455598}
MEASURED_TRAFFIC_OTHER = {"scaled_fp16_4096^3": 84835801, "quantize_pack_fp16_4096x4096": 42113123}


def roofline_of(m, n, k, bound, ms):
    ops = 2.0 * m * n * k
    if bound == "mfma":
        achieved = ops / ms / 1e9  # TOP/s
        return {"bound": "mfma", "achieved": round(achieved, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                "frac": round(achieved / INT8_PEAK_TOPS, 4), "traffic": MEASURED_TRAFFIC.get((m, n, k))}
    achieved = algorithmic_bytes(m, n, k) / ms / 1e6  # GB/s
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get((m, n, k))}


def run_workload(name, steps, warmup, check_rows=64):
    import numpy as np
    import torch

    import quadmul            # the drop-in extension module
    import quadmul_amd as qm  # config introspection only

    row, m, n, k, bound = WORKLOADS[name]
    ap, bp = make_packed(m, n, k, SEED_BASE + row)
    dev = torch.device("cuda:0")
    a_d, b_d = ap.to(dev), bp.to(dev)
    c_d = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    fn = lambda: quadmul.gemm(a_d, b_d, c_d, m, n, k)
    fn()
    torch.cuda.synchronize()
    graph_ms = time_graph(fn)   # also brings the clocks up before the timed steps
    wall_ms, event_ms = time_steps(fn, steps, warmup)
    kernel_ms = min(event_ms, graph_ms)
    rotating_ms = None
    if bound == "hbm":
        # Launched again and again on the same 8 MiB of B, the kernel reads B out of the L2 and
        # the 256 MiB memory-side cache, not HBM.  For the HBM roofline the launches of the
        # graph therefore rotate over enough copies of B (and their own C) to exceed that cache.
        ncopies = max(2, -(-(320 << 20) // max(1, bp.numel())))
        bs = [b_d] + [b_d.clone() for _ in range(ncopies - 1)]
        cs = [c_d] + [torch.empty_like(c_d) for _ in range(ncopies - 1)]
        turn = [0]

        def fn_rot():
            i = turn[0] % ncopies
            turn[0] += 1
            quadmul.gemm(a_d, bs[i], cs[i], m, n, k)

        rotating_ms = time_graph(fn_rot, launches=5 * ncopies)
        for c_i in cs[1:]:
            assert torch.equal(c_i, c_d)
        del bs, cs
    scaled_ms = None
    if name == "square4096":
        # the same GEMM with the dequantising epilogue fused in (fp16 out): less than half the bytes
        rs = torch.rand(m, device=dev) * 0.02 + 1e-3
        cs = torch.rand(n, device=dev) * 0.05 + 1e-4
        d_d = torch.empty((m, n), dtype=torch.float16, device=dev)
        fn_s = lambda: quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
        fn_s()
        torch.cuda.synchronize()
        scaled_ms = time_graph(fn_s)
        want = ((c_d.to(torch.float32) * rs[:, None]) * cs[None, :]).to(torch.float16)
        assert torch.equal(d_d.view(torch.int16), want.view(torch.int16)), "scaled output differs from its definition"
    out = {
        "workload": f"{name}: M={m} N={n} K={k}, signed int4 packed 2/byte along K (low nibble = even k), "
                    f"C=A.B^T int32, uniform [-8,7] seed {hex(SEED_BASE + row)}",
        "m": m, "n": n, "k": k,
        "kernel": qm.config_name(qm.select_config(m, n, k) & 0xFFFF),
        "ms_per_step_wall": round(wall_ms, 5), "ms_per_step_events": round(event_ms, 5), "ms_per_launch_graph": round(graph_ms, 5),
        "tops": round(2.0 * m * n * k / wall_ms / 1e9, 2),           # whole-job rate over the timed steps
        "tops_kernel": round(2.0 * m * n * k / kernel_ms / 1e9, 2),  # from the per-launch duration
        "gbs_algorithmic": round(algorithmic_bytes(m, n, k) / kernel_ms / 1e6, 1),
        "roofline": roofline_of(m, n, k, bound, kernel_ms if rotating_ms is None else rotating_ms),
    }
    if scaled_ms is not None:
        out["scaled_fp16_output"] = {"entry_point": "quadmul.gemm_scaled(a, b, d, m, n, k, row_scale, col_scale)",
                                     "ms_per_launch_graph": round(scaled_ms, 5), "tops": round(2.0 * m * n * k / scaled_ms / 1e9, 1),
                                     "frac_of_int8_peak": round(2.0 * m * n * k / scaled_ms / 1e9 / INT8_PEAK_TOPS, 4),
                                     "algorithmic_bytes": m * k // 2 + n * k // 2 + 2 * m * n + 4 * (m + n),
                                     "traffic": MEASURED_TRAFFIC_OTHER["scaled_fp16_4096^3"],
                                     "checked": "every element against torch's float32 arithmetic on the int32 result"}
    if rotating_ms is not None:
        out["ms_per_launch_graph_rotating_b"] = round(rotating_ms, 5)
        out["roofline"]["note"] = "launches rotate over copies of B exceeding the 256 MiB memory-side cache: B comes from HBM"
        out["roofline_b_cache_resident"] = roofline_of(m, n, k, bound, kernel_ms)
    return out, (ap, bp, c_d, m, n, k, wall_ms)


def cpu_baseline(ap, bp, c_gpu, m, n, k):
    """The CPU oracle (a restatement of the reference's cpu_gemm_int8) on a bounded sample
    of the same workload: a block of rows of A against all of B; also checks the GPU result
    for those rows bit-exactly."""
    import numpy as np

    import oracle

    threads = oracle.max_threads()
    # budgets in MACs: about 10 s on all cores, about 10 s on one core (measured rates:
    # ~1.5e10 MAC/s per core); at 4096^3 the first covers every row of A
    rows_mt = min(m, max(16, int(1.5e10 * 10 * min(threads, 8) / (n * k))))
    rows_1t = min(m, max(4, int(1.5e10 * 10 / (n * k))))
    sel_mt = np.linspace(0, m - 1, rows_mt).astype(np.int32)
    t0 = time.perf_counter()
    c_mt = oracle.gemm_i4_rows(ap.numpy(), bp.numpy(), sel_mt, threads=0)
    t_mt = time.perf_counter() - t0
    sel_1t = sel_mt[:rows_1t]
    t0 = time.perf_counter()
    c_1t = oracle.gemm_i4_rows(ap.numpy(), bp.numpy(), sel_1t, threads=1)
    t_1t = time.perf_counter() - t0
    got = c_gpu.cpu().numpy()
    exact = bool((got[sel_mt] == c_mt).all() and (got[sel_1t] == c_1t).all())
    tops_mt = 2.0 * rows_mt * n * k / t_mt / 1e12
    tops_1t = 2.0 * rows_1t * n * k / t_1t / 1e12
    return {
        "value": round(tops_mt, 5), "unit": "TOPS", "cores": threads, "kind": "port",
        "sample": f"{rows_mt} of {m} rows of A (evenly spaced) x all {n} rows of B, K={k}; unpack + triple loop "
                  f"as kernel.cu:291-306,389-408, OpenMP over rows, {t_mt:.2f} s",
        "single_thread": {"value": round(tops_1t, 5), "unit": "TOPS", "cores": 1,
                          "sample": f"{rows_1t} rows, the reference's loop nest unchanged, {t_1t:.2f} s"},
        "gpu_rows_bit_exact": exact,
    }


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="square4096", choices=sorted(WORKLOADS) + ["square4096_scaled_f16", "quantize4096_f16"],
                    help="the workload of the JSON line; the last two names exist for --launches-only (profiling) only")
    ap.add_argument("--no-targets", action="store_true", help="skip the other target shapes")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--launches-only", type=int, default=0, metavar="N",
                    help="profiling aid: just N launches of --workload (after one warm-up), nothing else")
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
    if a.launches_only and a.workload == "quantize4096_f16":
        import quadmul

        x = torch.randn((4096, 4096), device="cuda:0").to(torch.float16)
        for _ in range(a.launches_only + 1):
            quadmul.quantize_pack(x)
        torch.cuda.synchronize()
        print(json.dumps({"launches_only": a.launches_only, "workload": a.workload}))
        return 0
    if a.launches_only and a.workload == "square4096_scaled_f16":
        import quadmul

        row, m, n, k, _ = WORKLOADS["square4096"]
        apk, bpk = make_packed(m, n, k, SEED_BASE + row)
        a_d, b_d = apk.to("cuda:0"), bpk.to("cuda:0")
        d_d = torch.empty((m, n), dtype=torch.float16, device="cuda:0")
        rs, cs = torch.rand(m, device="cuda:0") * 0.02 + 1e-3, torch.rand(n, device="cuda:0") * 0.05 + 1e-4
        for _ in range(a.launches_only + 1):
            quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
        torch.cuda.synchronize()
        print(json.dumps({"launches_only": a.launches_only, "workload": a.workload}))
        return 0
    if a.workload not in WORKLOADS:
        print("bench.py: that workload name is for --launches-only", file=sys.stderr)
        return 2
    if a.launches_only:
        import quadmul

        row, m, n, k, _ = WORKLOADS[a.workload]
        apk, bpk = make_packed(m, n, k, SEED_BASE + row)
        a_d, b_d = apk.to("cuda:0"), bpk.to("cuda:0")
        c_d = torch.empty((m, n), dtype=torch.int32, device="cuda:0")
        for _ in range(a.launches_only + 1):
            quadmul.gemm(a_d, b_d, c_d, m, n, k)
        torch.cuda.synchronize()
        print(json.dumps({"launches_only": a.launches_only, "workload": a.workload}))
        return 0

    main_res, (apk, bpk, c_d, m, n, k, wall_ms) = run_workload(a.workload, a.steps, a.warmup)
    line = {
        "metric": "int4 GEMM TOPS and % of int8 MFMA peak / % HBM BW, 1xMI355X",
        "value": main_res["tops"], "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": main_res["ms_per_step_wall"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8 (s4 nibbles widened to 16*s4) x i8 -> i32 MFMA, exact",
        "data": "synthetic",
        "config": {"workload": main_res["workload"], "kernel": main_res["kernel"], "entry_point": "quadmul.gemm(a, b, c, m, n, k)",
                   "ms_per_step_events": main_res["ms_per_step_events"], "ms_per_launch_graph": main_res["ms_per_launch_graph"]},
        "roofline": main_res["roofline"],
    }
    if "scaled_fp16_output" in main_res:
        line["scaled_fp16_output"] = main_res["scaled_fp16_output"]
    if a.workload == "square4096":
        # the step before the GEMM: quantise + pack a [4096, 4096] fp16 activation matrix (HBM-bound)
        import quadmul
        x = torch.randn((m, k), device="cuda:0").to(torch.float16)
        q_ms = time_graph(lambda: quadmul.quantize_pack(x), launches=50)
        q_bytes = m * k * 2 + m * k // 2 + 4 * m
        line["quantize_pack_fp16"] = {"entry_point": "quadmul.quantize_pack(x)", "rows": m, "k": k, "ms_per_launch_graph": round(q_ms, 5),
                                      "algorithmic_bytes": q_bytes,
                                      "roofline": {"bound": "hbm", "achieved": round(q_bytes / q_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                                   "frac": round(q_bytes / q_ms / 1e6 / HBM_PEAK_GBS, 4),
                                                   "traffic": MEASURED_TRAFFIC_OTHER["quantize_pack_fp16_4096x4096"]}}
        del x
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(apk, bpk, c_d, m, n, k)
    del apk, bpk, c_d
    if not a.no_targets:
        targets = []
        for name in sorted(WORKLOADS):
            if name == a.workload:
                continue
            res, _ = run_workload(name, max(20, a.steps // 2), a.warmup)
            targets.append({kk: res[kk] for kk in ("workload", "kernel", "tops", "tops_kernel", "gbs_algorithmic", "ms_per_step_events",
                                                   "ms_per_launch_graph", "ms_per_launch_graph_rotating_b", "roofline",
                                                   "roofline_b_cache_resident") if kk in res})
        line["targets"] = targets
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
