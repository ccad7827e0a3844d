"""Every row of the tuned per-shape table (csrc/qm_tile_table.inc: the reference's dispatch
list, kernel.cu:343-384, plus the contract's shapes) through the drop-in entry point
``quadmul.gemm``: the whole product against the CPU oracle up to 512 rows, every element
against an exact fp32 product and sampled rows against the oracle above that.  A retuned
row that breaks is caught here, not only by the benchmark table.  And a process whose very
first call of a configuration happens inside HIP graph capture."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import SEED_BASE, poisoned_c

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def table_rows():
    text = open(os.path.join(ROOT, "quadmul_amd", "csrc", "qm_tile_table.inc")).read()
    rows = [(int(m), int(n), int(k), name) for m, n, k, name in re.findall(r'^\{(\d+), (\d+), (\d+), "([^"]+)"', text, flags=re.M)]
    assert len(rows) >= 52
    return rows


ROWS = table_rows()
FAMILIES = sorted({(n, k) for _, n, k, _ in ROWS})


def unpack_on_gpu(p):
    """[rows, K/2] packed bytes -> [rows, K] fp32 values, in torch arithmetic (not the library's kernel)."""
    lo = (p << 4).view(torch.int8) >> 4      # low nibble, sign-extended
    hi = p.view(torch.int8) >> 4             # high nibble, sign-extended
    return torch.stack((lo, hi), dim=2).reshape(p.shape[0], -1).float()


@pytest.mark.parametrize("family", FAMILIES, ids=lambda f: f"N{f[0]}_K{f[1]}")
def test_every_table_row_through_the_drop_in(oracle_mod, family):
    import quadmul

    n, k = family
    g = torch.Generator().manual_seed(SEED_BASE + 9000 + n + k)
    bp = torch.randint(-128, 128, (n, k // 2), dtype=torch.int8, generator=g)   # uniform bytes = uniform nibbles
    b_d = bp.to(DEV)
    b_f = unpack_on_gpu(b_d.view(torch.uint8))
    for (m, n_, k_, name) in ROWS:
        if (n_, k_) != family:
            continue
        print(f"  table row {m}x{n}x{k} ({name})", flush=True)
        assert qm.config_name(qm.select_config(m, n, k) & 0xFFFF) == name
        ap = torch.randint(-128, 128, (m, k // 2), dtype=torch.int8, generator=g)
        a_d = ap.to(DEV)
        c_d = poisoned_c(m, n, DEV)
        quadmul.gemm(a_d, b_d, c_d, m, n, k)
        torch.cuda.synchronize()
        if m <= 512:
            want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
            bad = oracle_mod.compare(c_d.cpu().numpy(), want)
            assert bad == -1, f"{m}x{n}x{k} ({name}): first mismatch at flat index {bad}"
        else:
            a_f = unpack_on_gpu(a_d.view(torch.uint8))
            for i in range(0, m, 1024):   # exact: every partial sum is an integer below 2^24
                exact = (a_f[i:i + 1024] @ b_f.t()).to(torch.int32)
                assert torch.equal(c_d[i:i + 1024], exact), f"{m}x{n}x{k} ({name}): rows {i}.. differ from the exact fp32 product"
                del exact
            rows = np.unique(np.linspace(0, m - 1, 6).astype(np.int32))
            want = oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)
            assert (c_d[rows.tolist()].cpu().numpy() == want).all(), f"{m}x{n}x{k} ({name}): sampled rows differ from the oracle"
            del a_f
        del a_d, c_d


COLD_CAPTURE = r"""
import sys
sys.path.insert(0, {root!r})
import torch
import quadmul            # nothing of the library has run in this process yet
if {with_init!r}:
    import quadmul_amd
    quadmul_amd.init()    # qm_init: every kernel's one-off set-up, no launch

dev = "cuda:0"
def unpack(p):
    lo = (p << 4).view(torch.int8) >> 4
    hi = p.view(torch.int8) >> 4
    return torch.stack((lo, hi), dim=2).reshape(p.shape[0], -1).float()
shapes = {shapes!r}
ops = []
gen = torch.Generator().manual_seed(1234)
for (m, n, k) in shapes:
    a = torch.randint(-128, 128, (m, k // 2), dtype=torch.int8, generator=gen).to(dev)
    b = torch.randint(-128, 128, (n, k // 2), dtype=torch.int8, generator=gen).to(dev)
    c = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=dev)
    ops.append((a, b, c, m, n, k))
torch.cuda.synchronize()
side = torch.cuda.Stream()
side.wait_stream(torch.cuda.current_stream())
graph = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
        for (a, b, c, m, n, k) in ops:
            quadmul.gemm(a, b, c, m, n, k)     # the first call of each configuration: under capture
torch.cuda.current_stream().wait_stream(side)
for replay in range(3):
    for (a, b, c, m, n, k) in ops:
        c.fill_(0x7F7F7F7F)
    graph.replay()
    torch.cuda.synchronize()
    for (a, b, c, m, n, k) in ops:
        want = (unpack(a.view(torch.uint8)) @ unpack(b.view(torch.uint8)).t()).to(torch.int32)
        assert torch.equal(c, want), (replay, m, n, k)
print("COLD-CAPTURE-OK")
"""


@pytest.mark.parametrize("with_init", [False, True], ids=["cold", "after_qm_init"])
def test_first_call_of_a_configuration_inside_graph_capture(with_init):
    """A fresh process whose first use of the library is a captured launch: the kernels' one-off
    set-up (LDS size attribute, residency query, scratch address) must work there -- or have
    been done by qm_init beforehand -- and the replays must be exact.  One shape per kernel family, a K split through the workspace
    included."""
    shapes = [(1024, 1024, 1024), (512, 768, 2048 + 32), (640, 4096, 20480), (128, 4096, 14336), (16, 4096, 4096), (40, 512, 1024), (1, 512, 4096), (33, 70, 30)]
    names = {qm.config_name(qm.select_config(m, n, k) & 0xFFFF)[0] for (m, n, k) in shapes}
    assert {"q", "p", "d", "v", "g"} <= names, names
    assert (qm.select_config(640, 4096, 20480) >> 24) & 0x3F > 1     # the K split through the workspace
    code = COLD_CAPTURE.format(root=ROOT, shapes=shapes, with_init=with_init)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0 and "COLD-CAPTURE-OK" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
