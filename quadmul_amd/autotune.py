"""Autotuner for the per-shape kernel table (``csrc/qm_tile_table.inc``).

The reference's table (configs.cu:19-689) was produced by a tuner that was never
published (its ``tuning/`` directory is git-ignored, README.md:13).  This one
times every compiled-in configuration that supports a shape, over a few raster
group heights, on the GPU it runs on, checks each candidate bit-exactly against
the library's own generic kernel, and writes the winners as table rows.

    python -m quadmul_amd.autotune --shapes named --json out.json --emit table.inc

Timing: HIP events on the stream the kernels are launched on, back-to-back
launches for at least ``--min-ms`` per sample, median of ``--reps`` samples.
"""
from __future__ import annotations

import argparse
import json
import re
import sys
import time
from typing import Dict, Iterable, List, Tuple

import torch

import quadmul_amd as qm

NAMED_SHAPES: List[Tuple[int, int, int]] = [
    (1024, 1024, 1024), (4096, 4096, 4096),
    (1, 4096, 4096), (16, 4096, 4096), (64, 4096, 4096),
    (2048, 11008, 4096), (2048, 4096, 11008), (2048, 12288, 4096),
    (8192, 8192, 8192), (8000, 8000, 8064),
]

# The 42 shapes of the reference's dispatch chain (kernel.cu:343-384).
REFERENCE_SHAPES: List[Tuple[int, int, int]] = [
    (m, n, k)
    for (n, k) in [(57344, 8192), (8192, 8192), (28672, 4096), (10240, 8192), (6144, 4096), (8192, 28672), (4096, 14336)]
    for m in (128, 256, 512, 1024, 2048, 4096)
]

INT8_PEAK_TOPS = 5033.2   # 256 CU x 8192 int8 op/clk/CU x 2.4 GHz (dense)
HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(m: int, n: int, k: int) -> int:
    return m * k // 2 + n * k // 2 + 4 * m * n


def time_launches(fn, min_ms: float = 20.0, reps: int = 3, warmup: int = 5, graph: bool = True) -> float:
    """Median over ``reps`` of the mean time per launch, in ms.

    With ``graph`` the launches are captured into a HIP graph first (as the reference's
    harness does, test.py:78-91), so that the host's per-call cost -- several microseconds
    through Python -- does not bound what is measured for short kernels."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    fn()
    stop.record()
    stop.synchronize()
    one = max(start.elapsed_time(stop), 2e-3)
    if graph:
        inner = max(4, min(400, int(2.0 / one) + 1))   # about 2 ms of work per replay
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for _ in range(inner):
                    fn()
        torch.cuda.current_stream().wait_stream(side)
        run, per = g.replay, inner
        run()
        torch.cuda.synchronize()
    else:
        run, per = fn, 1
    iters = max(2, min(20000, int(min_ms / (one * per)) + 1))
    samples = []
    for _ in range(reps):
        start.record()
        for _ in range(iters):
            run()
        stop.record()
        stop.synchronize()
        samples.append(start.elapsed_time(stop) / (iters * per))
    samples.sort()
    return samples[len(samples) // 2]


def random_packed(rows: int, k: int, seed: int, device) -> torch.Tensor:
    g = torch.Generator(device="cpu").manual_seed(seed)
    # any byte is a valid pair of nibbles; uniform bytes = uniform int4 values
    return torch.randint(-128, 128, (rows, k // 2), dtype=torch.int8, generator=g).to(device)


def tune_shape(m: int, n: int, k: int, device, group_ms: Iterable[int], min_ms: float, reps: int, verbose: bool,
               only: str = "", rotate_mib: int = 0) -> Dict:
    """Time every configuration that takes the shape.  ``rotate_mib`` > 0: the timed launches
    rotate over as many copies of B (each with its own C) as fill that many MiB, so that B
    comes from HBM and not from the L2s and the 256 MiB memory-side cache -- what a weight
    matrix does in a model of many layers; 0 times all launches on one B, as the reference's
    harness does (test.py:78-91)."""
    a = random_packed(m, k, 1, device)
    b = random_packed(n, k, 2, device)
    c = torch.empty((m, n), dtype=torch.int32, device=device)
    ncopies = max(1, -(-(rotate_mib << 20) // max(1, b.numel()))) if rotate_mib > 0 else 1
    bs = [b] + [b.clone() for _ in range(ncopies - 1)]
    cs = [c] + [torch.empty_like(c) for _ in range(ncopies - 1)]
    # Cross-check: the generic kernel where it finishes quickly, else the first candidate
    # (parity against the CPU oracle is the test-suite's job, not the tuner's).
    ref = None
    if m * n * k <= 1 << 33:
        ref = torch.empty_like(c)
        qm.gemm_cfg(a, b, ref, m, n, k, qm.config_id("generic"))
    ops = 2.0 * m * n * k
    results = []
    for cfg, name in enumerate(qm.config_names()):
        if name == "generic" or not qm.config_supports(cfg, m, n, k):
            continue
        if only and not re.search(only, name):
            continue
        gms = list(group_ms) if name[0] in "tq" else [1]
        # K split (pipelined kernel only): worth trying when the tiles alone cannot fill the GPU
        kss = [1]
        tiles = 0
        if name[0] == "q":
            bm, bn = (int(x) for x in name[1:].split("_")[0].split("x"))
            tiles = -(-m // bm) * -(-n // bn)
            kss = [ks for ks in (1, 2, 3, 4, 6, 8, 12, 16) if ks == 1 or (tiles * ks <= 1024 and tiles <= 256 and (k // 128) // ks >= 4)]
        # (K split, group height, one-item-per-workgroup flag); the flag only changes the launch
        # when there are more work items than the device holds workgroups of the pipelined kernel
        variants = [(g_, k_, 0) for k_ in kss for g_ in (gms if k_ == 1 else gms[:1])]
        if name[0] == "q" and tiles > 256:
            variants += [(g_, 1, 1) for g_ in gms]
        for gm, ks, spread in variants:
            code = cfg | (gm << 16) | (ks << 24) | (spread << 30)
            c.fill_(0x7F7F7F7F)
            qm.gemm_cfg(a, b, c, m, n, k, code)
            if ref is None:
                ref = c.clone()
            if not torch.equal(c, ref):
                raise RuntimeError(f"{name} group_m={gm} ksplit={ks} spread={spread} disagrees with the cross-check result on {m}x{n}x{k}")
            turn = [0]

            def launch():
                i = turn[0] % ncopies
                turn[0] += 1
                qm.gemm_cfg(a, bs[i], cs[i], m, n, k, code)

            ms = time_launches(launch, min_ms, reps)
            results.append({"config": name, "group_m": gm, "ksplit": ks, "spread": spread, "ms": ms, "tops": ops / ms / 1e9,
                            "gbs": algorithmic_bytes(m, n, k) / ms / 1e6})
            if verbose:
                print(f"  {m}x{n}x{k} {name:28s} gm={gm:2d} ks={ks} spread={spread} {ms*1e3:9.1f} us {ops/ms/1e9:8.1f} TOPS", flush=True)
    results.sort(key=lambda r: r["ms"])
    best = results[0]
    print(f"{m}x{n}x{k}: best {best['config']} gm={best['group_m']} ks={best['ksplit']} spread={best['spread']} {best['ms']*1e3:.1f} us "
          f"{best['tops']:.1f} TOPS ({100*best['tops']/INT8_PEAK_TOPS:.1f}% int8 peak) "
          f"{best['gbs']:.0f} GB/s ({100*best['gbs']/HBM_PEAK_GBS:.1f}% HBM)", flush=True)
    out = {"m": m, "n": n, "k": k, "best": best, "all": results}
    if best["ksplit"] > 1:
        # The best choice splits K through a workspace.  Callers of the bare seven-argument
        # entry point have none: their row gets a second choice, the best unsplit one.  (An
        # unsplit launch runs the same with and without a workspace, so the times above hold;
        # a K split whose partial sums meet in C through atomics was measured behind the best
        # unsplit configuration on every shape of the reference's table.)
        nows = next(r for r in results if r["ksplit"] == 1)
        out["best_without_workspace"] = nows
        print(f"    without a workspace: {nows['config']} gm={nows['group_m']} {nows['ms']*1e3:.1f} us", flush=True)
    return out


def emit_table(tuned: List[Dict], path: str) -> None:
    lines = [
        "// Per-shape kernel choice measured on MI355X: {M, N, K, \"config name\", group_m, ksplit,",
        "// one item per workgroup[, \"config name\" and group_m for calls without a workspace, on rows",
        "// whose first choice splits K through one]}.",
        "// Written by quadmul_amd/autotune.py; shapes not listed use the cost model in",
        "// qm_select.hpp.  Counterpart of the reference's A40 table (configs.cu:19-689).",
    ]
    for t in tuned:
        b = t["best"]
        nows = t.get("best_without_workspace")
        extra = f", \"{nows['config']}\", {nows['group_m']}" if nows else ""
        note = f" ({nows['ms']*1e3:.1f} us without a workspace)" if nows else ""
        lines.append(f"{{{t['m']}, {t['n']}, {t['k']}, \"{b['config']}\", {b['group_m']}, {b['ksplit']}, {b.get('spread', 0)}{extra}}},  // {b['ms']*1e3:.1f} us, {b['tops']:.0f} TOPS{note}")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def parse_shapes(spec: str) -> List[Tuple[int, int, int]]:
    if spec in ("named", "baseline"):
        return NAMED_SHAPES
    if spec == "reference":
        return REFERENCE_SHAPES
    if spec == "all":
        return NAMED_SHAPES + REFERENCE_SHAPES
    out = []
    for part in spec.split(","):
        m, n, k = (int(x) for x in part.lower().split("x"))
        out.append((m, n, k))
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shapes", default="named", help="named | reference | all | MxNxK[,MxNxK...]")
    ap.add_argument("--group-m", default="1,2,4,8,16", help="raster group heights to try for tile kernels")
    ap.add_argument("--min-ms", type=float, default=20.0)
    ap.add_argument("--reps", type=int, default=3)
    ap.add_argument("--json", default=None, help="write all measurements here")
    ap.add_argument("--emit", default=None, help="write the table rows here (csrc/qm_tile_table.inc format)")
    ap.add_argument("--only", default="", help="regular expression: time only configurations whose name matches")
    ap.add_argument("--rotate-b", type=int, default=0, metavar="MiB",
                    help="rotate the timed launches over copies of B filling this many MiB (e.g. 320: B then comes from HBM)")
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("autotune needs a GPU", file=sys.stderr)
        return 2
    device = torch.device("cuda:0")
    gms = [int(x) for x in a.group_m.split(",")]
    t0 = time.time()
    tuned = [tune_shape(m, n, k, device, gms, a.min_ms, a.reps, a.verbose, a.only, a.rotate_b) for (m, n, k) in parse_shapes(a.shapes)]
    print(f"tuned {len(tuned)} shapes in {time.time()-t0:.0f} s on {torch.cuda.get_device_name(0)}", flush=True)
    if a.json:
        with open(a.json, "w") as f:
            json.dump({"device": torch.cuda.get_device_name(0), "library": qm.version(), "shapes": tuned}, f, indent=1)
    if a.emit:
        emit_table(tuned, a.emit)
    return 0


if __name__ == "__main__":
    sys.exit(main())
