"""Measurement probes (``quadmul_amd/lib/libqm_probe.so``, built from ``csrc/qm_probe.hip``):
what the part sustains, measured on the box, to set beside the nominal peaks.

    python -m quadmul_amd.probe          # prints one JSON object

* ``mfma_issue_peak``: a loop of independent ``v_mfma_i32_16x16x64_i8`` on 16*s4 operands
  (rotating over four operand register pairs, and on one pair for comparison),
  nothing else in the loop, on every SIMD of the device, timed between two events like the
  reference's harness times its kernel (kernel.cu:468-497).  One such MFMA is 32768 integer
  operations and issues in 16 cycles of a SIMD, so the rate also gives the clock the part
  sustains under that load.
* ``launch_floor``: an empty kernel, and a kernel that only reads 8 MiB, per launch inside a
  graph of back-to-back launches -- what any kernel on an 8 MiB operand pays before it
  computes anything.
"""
from __future__ import annotations

import ctypes
import json
import os
import statistics

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG, "lib", "libqm_probe.so")
_lib = None

INT8_PEAK_TOPS = 5033.2      # 256 CU x 8192 op/clk x 2.4 GHz
NOMINAL_MHZ = 2400.0


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f"{_LIB_PATH} is missing: build it with `python -m quadmul_amd.build`")
        lib = ctypes.CDLL(_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.qm_probe_mfma_issue.argtypes = [vp, ci, ci, ci, vp]
        lib.qm_probe_mfma_issue.restype = ctypes.c_double
        lib.qm_probe_empty.argtypes = [vp]
        lib.qm_probe_empty.restype = ci
        lib.qm_probe_read.argtypes = [vp, ctypes.c_size_t, vp, ci, ci, ci, vp]
        lib.qm_probe_read.restype = ci
        _lib = lib
    return _lib


def _mfma_issue_rate(lib, out, blocks, iters, pairs, seconds):
    """(TOP/s, ms per launch, warm-up launches) of the MFMA-only loop on `pairs` operand register pairs."""
    import torch

    stream = torch.cuda.current_stream().cuda_stream

    def launch():
        ops = lib.qm_probe_mfma_issue(out.data_ptr(), blocks, iters, pairs, stream)
        if ops < 0:
            raise RuntimeError(f"qm_probe_mfma_issue: hipError_t {int(-ops)}")
        return ops

    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ops = launch()
    torch.cuda.synchronize()
    e0.record()
    launch()
    e1.record()
    e1.synchronize()
    one = e0.elapsed_time(e1)
    n_warm = max(5, int(seconds * 1e3 / max(one, 1e-3)))
    for _ in range(n_warm):
        launch()
    times = []
    for _ in range(5):
        e0.record()
        launch()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    ms = statistics.median(times)
    return ops / ms / 1e9, ms, n_warm


def mfma_issue_peak(seconds: float = 0.6, blocks_per_cu: int = 1):
    """Sustained rate of the MFMA-only loop.  Launches of about 1.3 ms each, back to back
    for `seconds` (long enough for the power management to settle), the last five timed
    one by one: median.  Measured twice: with consecutive MFMAs rotating over four pairs of
    pseudo-random operand registers (``tops``: the operand buses toggle as they do in the
    GEMM) and with every MFMA on one pair (``tops_one_operand_pair``: they do not, so under a
    power cap this one is an upper bound)."""
    import torch

    lib = library()
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    blocks = cus * blocks_per_cu
    out = torch.zeros(2 * blocks, dtype=torch.int64, device=dev)
    iters = 12000   # x 16 MFMAs x 16 cycles = 3.07 M cycles: about 1.3 ms at 2.4 GHz
    tops1, ms1, _ = _mfma_issue_rate(lib, out, blocks, iters, 1, seconds)
    tops, ms, n_warm = _mfma_issue_rate(lib, out, blocks, iters, 4, seconds)
    counters = out.view(-1, 2).cpu()
    core, ref = int(counters[:, 0].max()), int(counters[:, 1].max())
    res = {
        "tops": round(tops, 1),
        "frac_of_nominal_int8_peak": round(tops / INT8_PEAK_TOPS, 4),
        # 16 cycles per MFMA and SIMD, every SIMD of every CU busy: rate / nominal rate x 2.4 GHz
        "implied_clock_mhz": round(tops / (INT8_PEAK_TOPS * cus / 256.0) * NOMINAL_MHZ, 0),
        "instruction": "v_mfma_i32_16x16x64_i8, operands 16*s4, 16 independent accumulators per wave, one wave per SIMD, "
                       "consecutive MFMAs on four different pairs of operand registers",
        "launch_ms_median_of_5": round(ms, 4), "warmup_launches": n_warm, "cus": cus,
        "tops_one_operand_pair": round(tops1, 1),
        "one_operand_pair": {"tops": round(tops1, 1), "frac_of_nominal_int8_peak": round(tops1 / INT8_PEAK_TOPS, 4),
                             "launch_ms_median_of_5": round(ms1, 4),
                             "note": "every MFMA reads the same two registers: the operand buses do not toggle (upper bound under a power cap)"},
        "method": "launches between two HIP events after the warm-ups (as kernel.cu:468-497)",
    }
    if ref > 0:
        # s_memtime ticks per 100 MHz reference tick: equals the core clock only where
        # s_memtime counts core cycles; reported as read
        res["memtime_per_100mhz_tick"] = round(core / ref, 3)
    return res


def launch_floor(read_bytes: int = 8 << 20, launches: int = 200, replays: int = 5, blocks: int = 512, threads: int = 256, lds_bytes: int = 0):
    """us per launch, inside a graph of back-to-back launches (median of the replays), of an
    empty kernel, of a kernel that reads `read_bytes` again and again from the same buffer
    (cache-fed) and of the same kernel rotating over copies that exceed the 256 MiB
    memory-side cache (HBM-fed)."""
    import torch

    lib = library()
    dev = torch.device("cuda:0")
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    ncopies = max(2, -(-(320 << 20) // read_bytes))
    bufs = [torch.randint(0, 255, (read_bytes,), dtype=torch.uint8, device=dev) for _ in range(ncopies)]

    def timed(fn, n):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            fn(0)
            with torch.cuda.graph(g, stream=side):
                for i in range(n):
                    fn(i)
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
            ts.append(e0.elapsed_time(e1) / n * 1e3)
        return statistics.median(ts)

    def st(i):
        return torch.cuda.current_stream().cuda_stream

    def chk(rc):
        if rc != 0:
            raise RuntimeError(f"probe launch failed: {rc}")

    empty = timed(lambda i: chk(lib.qm_probe_empty(st(i))), launches)
    hot = timed(lambda i: chk(lib.qm_probe_read(bufs[0].data_ptr(), read_bytes, sink.data_ptr(), blocks, threads, lds_bytes, st(i))), launches)
    cold = timed(lambda i: chk(lib.qm_probe_read(bufs[i % ncopies].data_ptr(), read_bytes, sink.data_ptr(), blocks, threads, lds_bytes, st(i))), 5 * ncopies)
    return {"empty_kernel_us": round(empty, 3), "read_only_us_cache_fed": round(hot, 3), "read_only_us_hbm_fed": round(cold, 3),
            "read_bytes": read_bytes, "read_launch": f"{blocks} workgroups x {threads} threads, {lds_bytes} bytes of LDS each", "read_only_gbs_hbm_fed": round(read_bytes / cold / 1e3, 1),
            "method": f"per launch inside a HIP graph of back-to-back launches, median of {replays} replays; "
                      f"HBM-fed: rotating over {ncopies} buffers (> 256 MiB)"}


def main():
    print(json.dumps({"mfma_issue_peak": mfma_issue_peak(), "launch_floor": launch_floor()}))


if __name__ == "__main__":
    main()
