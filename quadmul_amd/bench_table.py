"""Reproduces the reference's benchmark table on the GPU it runs on.

The reference's ``test.py`` (lines 18-126) times three things per (M, N, K) inside CUDA
graphs of 50 launches: ``torch._int_mm`` on the unpacked int8 operands (its "cuBLAS int8"
column), ``quadmul.gemm`` on the packed operands, and ``torch.matmul`` in fp16, and prints
TOPS = 2*M*N*K / t / 1e12 (test.py:110-113).  This script does the same with the drop-in
``quadmul`` module of this repository and writes a markdown table in the column layout of
the reference's ``benchmarks/a40.md``:

    python -m quadmul_amd.bench_table --out benchmarks/mi355x.md

Before timing, each shape is checked: the int4 result must equal the int8 library
result exactly (the reference accepts |diff| <= 1, test.py:41-43).

A second table times the same shapes through the bare seven-argument C entry point
``qm_gemm_i4`` -- the function a maintainer binds in place of the reference's ``wrapper``
(kernel.cu:334) -- which has no workspace to split K through, beside ``quadmul.gemm``, which
takes one from torch's allocator.
"""
from __future__ import annotations

import argparse
import sys

import torch

import quadmul_amd as qm
from quadmul_amd.autotune import INT8_PEAK_TOPS, REFERENCE_SHAPES, time_launches


def bench_shape(m: int, n: int, k: int, dev) -> dict:
    import quadmul

    g = torch.Generator().manual_seed(0x51AD0000 + m + n + k)
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=g).to(dev)
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=g).to(dev)
    a_p, b_p = quadmul.pack(a), quadmul.pack(b)          # device-side pack_b (test.py:6-15)
    c = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    c_ref = torch.empty((m, n), dtype=torch.int32, device=dev)
    bt = b.t()
    torch._int_mm(a, bt, out=c_ref)                      # the reference's oracle (test.py:39)
    quadmul.gemm(a_p, b_p, c, m, n, k)
    torch.cuda.synchronize()
    exact = bool(torch.equal(c, c_ref))
    a_h = torch.randn((m, k), dtype=torch.float16, device=dev)
    b_h = torch.randn((n, k), dtype=torch.float16, device=dev)
    c_h = torch.empty((m, n), dtype=torch.float16, device=dev)
    t_i8 = time_launches(lambda: torch._int_mm(a, bt, out=c_ref), 20.0, 3)
    t_i4 = time_launches(lambda: quadmul.gemm(a_p, b_p, c, m, n, k), 20.0, 3)
    # the bare C entry point: the same seven arguments as the reference's wrapper, no workspace
    lib = qm.library()
    c_bare = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)

    def bare():
        st = lib.qm_gemm_i4(a_p.data_ptr(), b_p.data_ptr(), c_bare.data_ptr(), m, n, k, torch.cuda.current_stream().cuda_stream)
        if st != 0:
            raise RuntimeError(f"qm_gemm_i4: status {st}")

    bare()
    torch.cuda.synchronize()
    exact = exact and bool(torch.equal(c_bare, c_ref))
    t_bare = time_launches(bare, 20.0, 3)
    t_f16 = time_launches(lambda: torch.matmul(a_h, b_h.t(), out=c_h), 20.0, 3)
    ops = 2.0 * m * n * k
    cfg = qm.select_config(m, n, k)
    cfg_bare = qm.select_config_ex(m, n, k, workspace=False)
    return {"m": m, "n": n, "k": k, "exact": exact, "kernel": qm.config_name(cfg & 0xFFFF), "ksplit": max(1, (cfg >> 24) & 0x3F),
            "kernel_bare": qm.config_name(cfg_bare & 0xFFFF), "ksplit_bare": max(1, (cfg_bare >> 24) & 0x3F),
            "int8": ops / t_i8 / 1e9, "int4": ops / t_i4 / 1e9, "fp16": ops / t_f16 / 1e9, "int4_bare": ops / t_bare / 1e9,
            "us": t_i4 * 1e3, "us_bare": t_bare * 1e3}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--out", default=None, help="markdown file to write (default: stdout only)")
    ap.add_argument("--min-m", type=int, default=128)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("bench_table needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    rows = []
    # the reference's row order: grouped by (N, K), M ascending (benchmarks/a40.md:5-37)
    order = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672), (6144, 4096), (28672, 4096), (4096, 14336)]
    for (n, k) in order:
        for (m, n2, k2) in sorted(s for s in REFERENCE_SHAPES if s[1] == n and s[2] == k):
            if m < a.min_m:
                continue
            r = bench_shape(m, n2, k2, dev)
            rows.append(r)
            print(f"{m}x{n2}x{k2}: int8 {r['int8']:.1f}  int4 {r['int4']:.1f}  fp16 {r['fp16']:.1f} TOPS  "
                  f"exact={r['exact']} kernel={r['kernel']}", flush=True)
    lines = [
        f"### Benchmark on {torch.cuda.get_device_name(0)} (MI355X, gfx950), torch {torch.__version__}",
        "",
        "Method of the reference's test.py:60-113 (graph-captured launches, TOPS = 2MNK/t); int8 = `torch._int_mm` "
        "(hipBLASLt), fp16 = `torch.matmul`; int4 = this repository's `quadmul.gemm`, checked bit-exact against the int8 "
        f"result before timing.  % of peak is against the dense int8 MFMA peak of {INT8_PEAK_TOPS:.1f} TOP/s.",
        "",
        "| M | N | K | hipBLASLt Int8 TOP/s | QuadMul Int4 TOP/s | hipBLASLt FP16 TOP/s | Speedup vs Int8 | Speedup vs FP16 | Int4 % of int8 peak | exact | kernel |",
        "|---|---|---|---|---|---|---|---|---|---|---|",
    ]
    for r in rows:
        lines.append(f"| {r['m']} | {r['n']} | {r['k']} | {r['int8']:.2f} | {r['int4']:.2f} | {r['fp16']:.2f} | "
                     f"{r['int4']/r['int8']:.2f}x | {r['int4']/r['fp16']:.2f}x | {100*r['int4']/INT8_PEAK_TOPS:.1f} | "
                     f"{'yes' if r['exact'] else 'NO'} | {r['kernel']} |")
    lines += [
        "",
        "### The same shapes through the bare entry point `qm_gemm_i4(A, B, C, m, n, k, stream)`",
        "",
        "`qm_gemm_i4` takes the seven arguments of the reference's `wrapper` (kernel.cu:334) and nothing else, so it has no "
        "workspace: where the table above splits K through one (K split > 1 there), it runs the cost model's choice without, "
        "partial sums meeting in C through integer atomics if it splits at all.  Same operands, same timing method, results "
        "checked bit-exact.  `qm_gemm_i4_ws` (a caller's workspace) and `qm_gemm_i4_static` (the library's own scratch array) "
        "run what `quadmul.gemm` runs.",
        "",
        "| M | N | K | quadmul.gemm us | K split | qm_gemm_i4 us | K split | qm_gemm_i4 / quadmul.gemm | qm_gemm_i4 TOP/s | kernel |",
        "|---|---|---|---|---|---|---|---|---|---|",
    ]
    for r in rows:
        lines.append(f"| {r['m']} | {r['n']} | {r['k']} | {r['us']:.1f} | {r['ksplit']} | {r['us_bare']:.1f} | {r['ksplit_bare']} | "
                     f"{r['us_bare']/r['us']:.2f}x | {r['int4_bare']:.2f} | {r['kernel_bare']} |")
    text = "\n".join(lines) + "\n"
    if a.out:
        with open(a.out, "w") as f:
            f.write(text)
    print(text)
    return 0 if all(r["exact"] for r in rows) else 1


if __name__ == "__main__":
    sys.exit(main())
