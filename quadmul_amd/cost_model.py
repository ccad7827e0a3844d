"""The fitted cost model behind the kernel choice for shapes outside the per-shape table
(``csrc/qm_cost_model.inc``, read by ``heuristic()`` in ``csrc/qm_select.hpp``).

The reference has no such fallback: a shape that is not one of the 42 of its dispatch chain
is skipped (kernel.cu:340-385).  Here every shape runs, and which kernel it runs on decides
how fast; the per-shape table covers the shapes that were tuned one by one, this model the
rest, from 33 rows up.

Model, per configuration c (a tile of the pipelined kernel, or a block of the wave-level
kernel, of bm x bn elements of C):

    items  = ceil(M / bm) * ceil(N / bn) * ksplit
    rounds = blend * ceil(items / slots) + (1 - blend) * max(1, items / slots)
    fill   = min(1, items / slots)
    ksteps = ceil(ceil(K / 128) / ksplit)
    us     = ksteps * (rounds * step_us + fill * busy_us) + rounds * round_us + launch_us
             [+ ksteps * rounds * skew_us                       when K % 256 != 0]
             [+ rounds * odd_us                                 when N % 4 != 0 and ksplit == 1]
             [+ max(1, ragged items / slots) * ragged_us        pipelined kernel, N % 4 == 0, ksplit == 1]
             [+ (ceil(M / bm) - 1) * N * K / 2e6 * reread_us    wave-level kernel, N * K / 2 > 32 MB, items > slots]
             [+ split_us + split_us_per_melem * ksplit * M * N / 1e6   when ksplit > 1]

``slots`` is the number of items the device works on at once (256 CUs, times the workgroups
of the configuration a CU holds where they do not slow each other down), ``blend`` says how
much a partly filled last round costs (1: as much as a full one -- one workgroup per CU;
towards 0: in proportion -- several small workgroups per CU, where the ones left speed up);
``busy_us`` is what a K-step slows down by as the device fills up (shared L2s, fabric and
power); ``odd_us`` is added per round when N % 4 != 0 (rows of C that are not 16-byte aligned:
the pipelined kernel then writes every tile after its last K-step, none of it folded into
that step); ``ragged_us`` per round of tiles that stick out of C (they are written through
guarded stores after the last K-step); ``reread_us`` per megabyte of B that the second and
later blocks of rows of the wave-level kernel read again after the L2s have lost it;
``skew_us`` is what a K-step costs more when the rows of A and B are not whole 128-byte
lines (K % 256 != 0: every 128-byte run of a row then lies across two cache lines -- 20 to 25 %
per step on the wave-level kernel, 6 to 15 % on the pipelined one).
The ten numbers per configuration and the two of the K split are least-squares fits
(relative error) to timings of every candidate on a few hundred random shapes:

    python -m quadmul_amd.cost_model collect --seed 11 --count 60 --domain large --data benchmarks/cost_model_data.jsonl
    python -m quadmul_amd.cost_model collect --seed 12 --count 60 --domain large --data benchmarks/cost_model_data.jsonl
    python -m quadmul_amd.cost_model collect --seed 13 --count 70 --domain small --data benchmarks/cost_model_data.jsonl
    python -m quadmul_amd.cost_model collect --seed 21 --count 60 --domain ragged --data benchmarks/cost_model_data.jsonl
    python -m quadmul_amd.cost_model collect --seed 22 --count 60 --domain ragged --data benchmarks/cost_model_data.jsonl
    python -m quadmul_amd.cost_model fit --data benchmarks/cost_model_data.jsonl --emit quadmul_amd/csrc/qm_cost_model.inc
    python -m quadmul_amd.cost_model check --data benchmarks/cost_model_data.jsonl      # the built library's choices

``collect`` needs the GPU (it appends to the data file); ``fit`` and ``check`` do not.
``check`` prints, for the choice the built library makes on every shape of the data, the
measured time of that choice over the best measured time of any candidate.
"""
from __future__ import annotations

import argparse
import json
import math
import random
import re
import sys
from typing import Dict, Iterable, List, Optional, Tuple

import numpy as np

# The configurations the model chooses among: the ones that are the fastest on some shapes of
# the data.  Left out: the same tile with another ring depth where that is never more than a
# percent or two ahead of its sibling, and configurations that win nowhere (they only add ways
# to be wrong).
CANDIDATES = [
    "q256x256_w2x2_s9o1", "q256x128_w2x2_s9o1", "q256x128_w2x2_s3o2", "q128x256_w2x2_s9o1", "q128x128_w2x2_s9o1",
    "q128x64_w2x2_s6o2", "q64x128_w2x2_s6o2", "q64x64_w2x2_s8o2",
    "d4x4_w8_r1", "d4x4_w4_r1", "d4x2_w8_r1", "d2x4_w8_r1", "d2x2_w8_r1", "d2x2_w1_r1", "d2x1_w16_r1", "d1x2_w8_r2", "d1x1_w4_r4",
]
SLOTS = (256, 512, 1024)
BLENDS = (0.0, 0.25, 0.5, 0.75, 1.0)

LARGE = dict(m=[72, 96, 128, 160, 200, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1280, 1536, 2048, 2560, 3072, 4096, 6144, 8192],
             n=[1024, 1536, 2048, 2560, 3072, 4096, 5120, 6144, 8192, 11008, 14336, 20480, 28672],
             k=[1024, 1536, 2048, 3072, 4096, 5120, 8192, 11008, 14336, 28672])
SMALL = dict(m=[33, 40, 48, 64, 65, 80, 100, 128, 192, 256, 384, 512, 1024, 2048, 4096, 8192, 16384],
             n=[256, 384, 512, 768, 1024, 1536, 2048, 4096, 8192, 16384],
             k=[128, 256, 384, 512, 768, 1024, 2048, 4096])


def block_of(name: str) -> Tuple[int, int]:
    """Rows and columns of C one work item of the configuration covers."""
    if name[0] == "q":
        bm, bn = (int(x) for x in name[1:].split("_")[0].split("x"))
        return bm, bn
    mm = re.match(r"d(\d+)x(\d+)_", name)
    return 16 * int(mm[1]), 16 * int(mm[2])


REREAD_BYTES = 32e6     # the eight L2s hold 32 MB between them


def features(name: str, m: int, n: int, k: int, ksplit: int, slots: int, blend: float) -> List[float]:
    bm, bn = block_of(name)
    rows, cols = -(-m // bm), -(-n // bn)
    items = rows * cols * ksplit
    rounds = blend * -(-items // slots) + (1.0 - blend) * max(1.0, items / slots)
    ksteps = -(-(-(-k // 128)) // ksplit)
    odd = rounds if (n % 4 and ksplit == 1) else 0.0
    ragged = reread = 0.0
    if name[0] == "q" and n % 4 == 0 and ksplit == 1:
        sticking_out = rows * cols - (m // bm) * (n // bn)
        if sticking_out:
            ragged = max(1.0, sticking_out / slots)
    if name[0] == "d" and n * k / 2 > REREAD_BYTES and items > slots:
        reread = (rows - 1) * n * k / 2e6
    skew = rounds * ksteps if k % 256 else 0.0
    return [rounds * ksteps, rounds, 1.0, min(1.0, items / slots) * ksteps, odd, ragged, reread, skew]


def load(paths: str) -> List[Dict]:
    """One shape per line; a line {"configs": [...]} names the configurations that the rows
    after it refer to by index (the names take most of the space otherwise)."""
    out = []
    for p in paths.split(","):
        names: List[str] = []
        for line in open(p):
            if not line.strip():
                continue
            row = json.loads(line)
            if "configs" in row:
                names = row["configs"]
                continue
            row["us"] = [[names[c] if isinstance(c, int) else c, ks, us] for c, ks, us in row["us"]]
            out.append(row)
    return out


def times_of(row: Dict) -> Dict[Tuple[str, int], float]:
    return {(name, int(ks)): us for name, ks, us in row["us"]}


def fit(rows: List[Dict], candidates: Iterable[str] = CANDIDATES) -> Dict:
    """Least squares on the relative error, per configuration over its unsplit timings, then
    the two numbers of the K split over what the split timings have beyond the unsplit model."""
    par: Dict[str, Dict] = {}
    for name in candidates:
        pts = [(r["m"], r["n"], r["k"], times_of(r)[(name, 1)]) for r in rows if (name, 1) in times_of(r)]
        if len(pts) < 8:
            continue
        y = np.array([p[3] for p in pts])
        best = None
        for slots in SLOTS:
            for blend in BLENDS:
                x = np.array([features(name, m, n, k, 1, slots, blend) for (m, n, k, _) in pts])
                coef = np.linalg.lstsq(x / y[:, None], np.ones_like(y), rcond=None)[0]
                err = float(np.sqrt(np.mean((x @ coef / y - 1.0) ** 2)))
                if best is None or err < best[0]:
                    best = (err, slots, blend, coef)
        par[name] = {"slots": best[1], "blend": best[2], "step_us": float(best[3][0]), "round_us": float(best[3][1]),
                     "launch_us": float(best[3][2]), "busy_us": float(best[3][3]), "odd_us": float(best[3][4]), "ragged_us": float(best[3][5]),
                     "reread_us": float(best[3][6]), "skew_us": float(best[3][7]), "rms": best[0], "points": len(pts)}
    xs, ys = [], []
    for r in rows:
        for (name, ks), us in times_of(r).items():
            if ks > 1 and name in par:
                xs.append([1.0, ks * r["m"] * r["n"] / 1e6])
                ys.append(us - predict(par, None, name, r["m"], r["n"], r["k"], 1, ksplit_items=ks))
    split = np.linalg.lstsq(np.array(xs), np.array(ys), rcond=None)[0] if xs else np.zeros(2)
    return {"configs": par, "split_us": float(split[0]), "split_us_per_melem": float(split[1])}


def predict(par: Dict, model: Optional[Dict], name: str, m: int, n: int, k: int, ksplit: int, ksplit_items: int = 0) -> float:
    p = par[name]
    ks = ksplit_items or ksplit
    f = features(name, m, n, k, ks, p["slots"], p["blend"])
    us = f[0] * p["step_us"] + f[1] * p["round_us"] + p["launch_us"] + f[3] * p["busy_us"] + f[4] * p["odd_us"] + f[5] * p["ragged_us"] + f[6] * p["reread_us"] + f[7] * p["skew_us"]
    if model is not None and ksplit > 1:
        us += model["split_us"] + model["split_us_per_melem"] * ksplit * m * n / 1e6
    return us


def choose(model: Dict, row: Dict) -> Tuple[str, int]:
    """The model's choice among the variants that were timed for the shape."""
    best = None
    for (name, ks) in times_of(row):
        if name not in model["configs"]:
            continue
        us = predict(model["configs"], model, name, row["m"], row["n"], row["k"], ks)
        if best is None or us < best[0]:
            best = (us, name, ks)
    return best[1], best[2]


def regret(rows: List[Dict], chooser) -> List[Tuple[float, int, int, int, str, int, str]]:
    """(time of the chosen variant / best time, M, N, K, chosen, its K split, best) per shape;
    shapes whose chosen variant was not timed are left out."""
    out = []
    for r in rows:
        t = times_of(r)
        name, ks = chooser(r)
        if (name, ks) not in t:
            continue
        best = min(t, key=t.get)
        out.append((t[(name, ks)] / t[best], r["m"], r["n"], r["k"], name, ks, best[0] + (f"/ks{best[1]}" if best[1] > 1 else "")))
    return sorted(out, reverse=True)


def summarise(label: str, reg: List[Tuple]) -> str:
    g = math.exp(sum(math.log(x[0]) for x in reg) / len(reg))
    return f"{label}: geomean {g:.4f} x the best measured, worst {reg[0][0]:.3f}, more than 5 % behind on {sum(x[0] > 1.05 for x in reg)} of {len(reg)} shapes"


def emit(model: Dict, path: str, rows: List[Dict]) -> None:
    reg = regret(rows, lambda r: choose(model, r))
    lines = [
        "// Fitted cost model of the kernel choice for shapes outside the per-shape table:",
        "// QM_COST(\"config name\", slots, blend, us per K-step of 128 and round, us per K-step with the device full,",
        "//         us per round, us more per round when N % 4 != 0, us per round of tiles that stick out of C,",
        "//         us per MB of B read again, us more per K-step and round when K % 256 != 0, us per launch)",
        "// and QM_COST_SPLIT(us per K split, us per million partial elements).  The formula is in",
        "// heuristic() (qm_select.hpp) and in quadmul_amd/cost_model.py, which wrote this file from",
        f"// timings of every candidate on {len(rows)} shapes on MI355X.",
        "// " + summarise("the model's choices on those shapes", reg),
    ]
    for name in CANDIDATES:
        p = model["configs"].get(name)
        if p:
            lines.append(f"QM_COST(\"{name}\", {p['slots']}, {p['blend']:.2f}f, {p['step_us']:.4f}f, {p['busy_us']:.4f}f, {p['round_us']:.3f}f, {p['odd_us']:.3f}f, {p['ragged_us']:.3f}f, {p['reread_us']:.4f}f, {p['skew_us']:.4f}f, {p['launch_us']:.3f}f)"
                         f"  // rms {100*p['rms']:.1f} % over {p['points']} shapes")
    lines.append(f"QM_COST_SPLIT({model['split_us']:.3f}f, {model['split_us_per_melem']:.4f}f)")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def sample_shapes(seed: int, count: int, domain: str) -> List[Tuple[int, int, int]]:
    rng = random.Random(seed)
    d = LARGE if domain == "large" else SMALL
    out: List[Tuple[int, int, int]] = []
    while len(out) < count:
        if domain == "ragged":
            # log-uniform, no multiples of anything but K's 32
            m = int(math.exp(rng.uniform(math.log(33), math.log(8192))))
            n = int(math.exp(rng.uniform(math.log(256), math.log(40000))))
            k = 32 * int(math.exp(rng.uniform(math.log(4), math.log(1000))))
        else:
            m, n, k = rng.choice(d["m"]), rng.choice(d["n"]), rng.choice(d["k"])
        if domain != "large" and m * n < 65536:
            continue
        if 2.0 * m * n * k > 1.2e12:      # (keeps a shape's candidates within seconds)
            continue
        out.append((m, n, k))
    return out


def collect(seed: int, count: int, domain: str, path: str) -> None:
    import torch

    import quadmul_amd as qm
    from quadmul_amd import autotune

    device = torch.device("cuda:0")
    names = qm.config_names()
    with open(path, "a") as f:
        f.write(json.dumps({"configs": names}, separators=(",", ":")) + "\n")
        for (m, n, k) in sample_shapes(seed, count, domain):
            r = autotune.tune_shape(m, n, k, device, [1, 4, 16], 6.0, 3, False)
            best: Dict[Tuple[str, int], float] = {}
            for x in r["all"]:
                if x["spread"] or x["config"][0] not in "dq":
                    continue
                key = (x["config"], x["ksplit"])
                best[key] = min(best.get(key, 1e30), x["ms"] * 1e3)     # (over the raster group heights)
            f.write(json.dumps({"m": m, "n": n, "k": k, "seed": seed,
                                "us": [[names.index(c), ks, round(us, 2)] for (c, ks), us in sorted(best.items())]}, separators=(",", ":")) + "\n")
            f.flush()


def library_choice(row: Dict) -> Tuple[str, int]:
    import quadmul_amd as qm

    code = qm.select_config(row["m"], row["n"], row["k"])
    return qm.config_name(code & 0xFFFF), max(1, (code >> 24) & 63)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=["collect", "fit", "check"])
    ap.add_argument("--data", required=True, help="JSON lines, one shape each (collect appends; fit and check read, comma-separated)")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--count", type=int, default=60)
    ap.add_argument("--domain", choices=["large", "small", "ragged"], default="large")
    ap.add_argument("--emit", default=None, help="fit: write csrc/qm_cost_model.inc here")
    a = ap.parse_args(argv)
    if a.what == "collect":
        collect(a.seed, a.count, a.domain, a.data)
        return 0
    rows = load(a.data)
    if a.what == "fit":
        model = fit(rows)
        for name, p in model["configs"].items():
            print(f"{name:22s} slots {p['slots']:4d} blend {p['blend']:.2f} step {p['step_us']:.4f} busy {p['busy_us']:.4f} round {p['round_us']:.2f} odd {p['odd_us']:.2f} ragged {p['ragged_us']:.2f} reread {p['reread_us']:.4f} skew {p['skew_us']:.4f} launch {p['launch_us']:.2f}"
                  f"  rms {100*p['rms']:.1f} %")
        print(f"K split: {model['split_us']:.2f} us + {model['split_us_per_melem']:.3f} us per million partial elements")
        reg = regret(rows, lambda r: choose(model, r))
        print(summarise("model", reg))
        if a.emit:
            emit(model, a.emit, rows)
        return 0
    reg = regret(rows, library_choice)
    for x in reg[:12]:
        print(f"  {x[0]:.3f}  {x[1]}x{x[2]}x{x[3]}: {x[4]}" + (f"/ks{x[5]}" if x[5] > 1 else "") + f", best {x[6]}")
    print(summarise("library", reg))
    return 0


if __name__ == "__main__":
    sys.exit(main())
