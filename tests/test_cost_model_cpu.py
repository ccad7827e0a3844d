"""The fitted cost model of the kernel choice (quadmul_amd/cost_model.py, csrc/qm_cost_model.inc):
the committed numbers are the fit of the committed timings, the built library evaluates the
same formula, and its choices stay close to the best measured candidate on every shape of
those timings.  The reference has no counterpart: it skips shapes outside its table
(kernel.cu:340-385).  No GPU: the timings are data, the choice is host code."""
import math
import os
import re

import quadmul_amd as qm
from quadmul_amd import cost_model as cm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DATA = os.path.join(ROOT, "benchmarks", "cost_model_data.jsonl")
INC = os.path.join(ROOT, "quadmul_amd", "csrc", "qm_cost_model.inc")


def _committed():
    text = open(INC).read()
    rows = {}
    for mm in re.finditer(r'^QM_COST\("([^"]+)", (\d+)((?:, [-\d.]+f){9})\)', text, re.M):
        rows[mm[1]] = (int(mm[2]),) + tuple(float(x.rstrip("f")) for x in mm[3].split(", ")[1:])
    sp = re.search(r"^QM_COST_SPLIT\(([-\d.]+)f, ([-\d.]+)f\)", text, re.M)
    return rows, (float(sp[1]), float(sp[2]))


def _tabled():
    text = open(os.path.join(ROOT, "quadmul_amd", "csrc", "qm_tile_table.inc")).read()
    return {tuple(int(x) for x in mm.groups()) for mm in re.finditer(r"^\{(\d+), (\d+), (\d+),", text, re.M)}


def test_the_committed_numbers_are_the_fit_of_the_committed_timings():
    rows = cm.load(DATA)
    assert len(rows) >= 300
    model = cm.fit(rows)
    inc, split = _committed()
    assert set(inc) == set(model["configs"]) == set(cm.CANDIDATES)
    for name, p in model["configs"].items():
        want = (p["slots"], p["blend"], p["step_us"], p["busy_us"], p["round_us"], p["odd_us"], p["ragged_us"], p["reread_us"], p["skew_us"], p["launch_us"])
        assert inc[name][0] == want[0] and all(abs(a - b) < 6e-4 for a, b in zip(inc[name][1:], want[1:])), (name, inc[name], want)
    assert abs(split[0] - model["split_us"]) < 6e-4 and abs(split[1] - model["split_us_per_melem"]) < 6e-5
    # every candidate is a configuration the library has
    assert all(name in qm.config_names() for name in cm.CANDIDATES)


def test_the_library_evaluates_the_same_formula():
    """Outside the per-shape table and the hand-written rules for up to 64 rows, the built
    library picks what the Python statement of the model picks (among the variants timed)."""
    rows = cm.load(DATA)
    model = cm.fit(rows)
    tabled = _tabled()
    checked = 0
    for r in rows:
        if r["m"] <= 64 or (r["m"], r["n"], r["k"]) in tabled:
            continue
        lib = cm.library_choice(r)
        mine = cm.choose(model, r)
        if lib != mine:
            # (a tie within the rounding of the committed numbers is no disagreement)
            a = cm.predict(model["configs"], model, lib[0], r["m"], r["n"], r["k"], lib[1])
            b = cm.predict(model["configs"], model, mine[0], r["m"], r["n"], r["k"], mine[1])
            assert abs(a - b) < 2e-3 * b, (r["m"], r["n"], r["k"], lib, mine, a, b)
        checked += 1
    assert checked >= 200


def test_the_choices_stay_close_to_the_best_measured_candidate():
    rows = cm.load(DATA)
    reg = cm.regret(rows, cm.library_choice)
    assert len(reg) >= 0.95 * len(rows)          # (the choice was among the timed variants)
    geomean = math.exp(sum(math.log(x[0]) for x in reg) / len(reg))
    assert geomean < 1.02, cm.summarise("library", reg)
    assert reg[0][0] < 1.4, reg[0]
    assert sum(x[0] > 1.05 for x in reg) <= 0.13 * len(reg), cm.summarise("library", reg)
    # shapes whose sizes are multiples of what the kernels work in (the first three collections)
    grid = [x for x in reg if x[1] % 8 == 0 and x[2] % 128 == 0 and x[3] % 128 == 0]
    assert len(grid) >= 180 and math.exp(sum(math.log(x[0]) for x in grid) / len(grid)) < 1.012
