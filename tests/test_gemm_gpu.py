"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle --
bit-exact, on seeded inputs, with C pre-poisoned to prove it is overwritten."""
import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import C_POISON, SEED_BASE, make_operands, pack_cpu, poisoned_c

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def run_gemm(ap, bp, m, n, k, cfg=qm.CFG_AUTO, workspace=True):
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    c_d = poisoned_c(m, n, DEV)
    qm.gemm_cfg(a_d, b_d, c_d, m, n, k, cfg, workspace)
    torch.cuda.synchronize()
    return c_d.cpu().numpy()


def fp32_matmul_on_gpu(a, b):
    """Exact for these sizes: every partial sum is an integer below 2^24."""
    a_d, b_d = a.to(DEV).float(), b.to(DEV).float()
    out = torch.empty((a.shape[0], b.shape[0]), dtype=torch.int32, device=DEV)
    for i in range(0, a.shape[0], 2048):
        out[i:i + 2048] = (a_d[i:i + 2048] @ b_d.t()).to(torch.int32)
    return out


SMALL_SHAPES = [
    (1, 1, 32), (1, 16, 64), (2, 15, 96), (15, 17, 128), (16, 16, 160), (17, 63, 256), (33, 65, 224),
    (63, 130, 512), (64, 64, 1024), (65, 255, 384), (127, 129, 640), (128, 256, 4096), (200, 300, 1184),
    (256, 256, 128), (257, 511, 288), (300, 70, 2080),
]


@pytest.mark.parametrize("shape", SMALL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_every_config_matches_oracle(oracle_mod, shape):
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 1000 + m * 7 + n * 3 + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not qm.config_supports(cfg, m, n, k):
            continue
        # raster group heights; K splits (pipelined kernel only: 3 does not divide the K-steps,
        # 8 leaves some splits empty on short K)
        variants = [(1, 1), (3, 1)] + ([(2, 2), (1, 3), (4, 8)] if name.startswith("q") else [])
        for gm, ks in variants:
            # a K split with a workspace (partial tiles, then a kernel that adds them up) and
            # without one (atomic adds into a zero-filled C)
            for ws in ([True, None] if ks > 1 else [True]):
                got = run_gemm(ap, bp, m, n, k, cfg | (gm << 16) | (ks << 24), ws)
                bad = oracle_mod.compare(got, want)
                assert bad == -1, (f"{name} group_m={gm} ksplit={ks} workspace={ws}: first mismatch at flat index {bad}: "
                                   f"got {got.flat[bad]} want {want.flat[bad]}")
        ran += 1
    assert ran >= 2
    got = run_gemm(ap, bp, m, n, k)
    assert oracle_mod.compare(got, want) == -1


GENERIC_SHAPES = [(1, 1, 2), (3, 5, 30), (17, 33, 34), (70, 33, 160 + 2), (100, 130, 510), (5, 130, 34)]


@pytest.mark.parametrize("shape", GENERIC_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_k_not_multiple_of_32_takes_generic_path(oracle_mod, shape):
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 2000 + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    assert qm.config_name(qm.select_config(m, n, k) & 0xFFFF) == "generic"
    assert oracle_mod.compare(run_gemm(ap, bp, m, n, k), oracle_mod.gemm_i4(ap.numpy(), bp.numpy())) == -1


def test_unaligned_operands_take_generic_path(oracle_mod):
    m, n, k = 37, 41, 128
    a, b = make_operands(m, n, k, SEED_BASE + 2100)
    ap, bp = pack_cpu(a), pack_cpu(b)
    buf_a = torch.zeros(ap.numel() + 16, dtype=torch.int8, device=DEV)
    buf_b = torch.zeros(bp.numel() + 16, dtype=torch.int8, device=DEV)
    a_d = buf_a[3:3 + ap.numel()].view(m, k // 2)
    b_d = buf_b[5:5 + bp.numel()].view(n, k // 2)
    a_d.copy_(ap)
    b_d.copy_(bp)
    c_d = poisoned_c(m, n, DEV)
    qm.gemm(a_d, b_d, c_d, m, n, k)
    assert oracle_mod.compare(c_d.cpu().numpy(), oracle_mod.gemm_i4(ap.numpy(), bp.numpy())) == -1


@pytest.mark.parametrize("name", ["gemm_i4_32x48x64", "gemm_i4_70x33x160", "gemm_i4_5x130x34"])
def test_golden_fixtures(name):
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", name + ".npz"))
    m, k = z["a"].shape
    n = z["b"].shape[0]
    got = run_gemm(torch.from_numpy(z["a_packed"]), torch.from_numpy(z["b_packed"]), m, n, k)
    assert (got == z["c"]).all()


def test_nibble_product_table_and_one_hot(oracle_mod):
    s4 = lambda v: v - 16 if v > 7 else v
    vals = torch.tensor([s4(i) for i in range(16)], dtype=torch.int8)
    k = 64
    for pos in (0, 1, 30, 31, 32, 33, 63):
        a = torch.zeros(16, k, dtype=torch.int8)
        a[:, pos] = vals
        got = run_gemm(pack_cpu(a), pack_cpu(a), 16, 16, k)
        assert (got == np.outer(vals.numpy().astype(np.int32), vals.numpy().astype(np.int32))).all(), pos
        b = torch.zeros(16, k, dtype=torch.int8)
        b[:, pos ^ 1] = vals
        assert (run_gemm(pack_cpu(a), pack_cpu(b), 16, 16, k) == 0).all(), pos


@pytest.mark.parametrize("shape", [(16, 64, 4096), (80, 272, 11008), (300, 260, 28672)], ids=lambda s: "x".join(map(str, s)))
def test_extremes_closed_form_on_every_config(shape):
    m, n, k = shape
    lo_a = pack_cpu(torch.full((m, k), -8, dtype=torch.int8))
    lo_b = pack_cpu(torch.full((n, k), -8, dtype=torch.int8))
    hi_b = pack_cpu(torch.full((n, k), 7, dtype=torch.int8))
    for cfg, name in enumerate(qm.config_names()):
        if not qm.config_supports(cfg, m, n, k) or name == "generic":
            continue
        assert (run_gemm(lo_a, lo_b, m, n, k, cfg) == 64 * k).all(), name   # largest positive accumulator
        assert (run_gemm(lo_a, hi_b, m, n, k, cfg) == -56 * k).all(), name  # most negative accumulator
        if name.startswith("q"):  # split K: partial sums meet in a workspace, or by atomic adds
            assert (run_gemm(lo_a, hi_b, m, n, k, cfg | (4 << 24)) == -56 * k).all(), name
            assert (run_gemm(lo_a, hi_b, m, n, k, cfg | (4 << 24), None) == -56 * k).all(), name


def test_largest_exact_k_and_beyond(oracle_mod):
    # K = 131040 is the largest multiple of 32 the x16 widening covers exactly; past it the
    # generic kernel must take over, with the same results.
    m, n = 16, 32
    for k in (131040, 131072):
        a = pack_cpu(torch.full((m, k), -8, dtype=torch.int8))
        b = pack_cpu(torch.full((n, k), -8, dtype=torch.int8))
        assert (run_gemm(a, b, m, n, k) == 64 * k).all(), k
    assert qm.config_name(qm.select_config(m, n, 131072) & 0xFFFF) == "generic"


def test_dtypes_and_overwrite(oracle_mod):
    m, n, k = 48, 80, 256
    a, b = make_operands(m, n, k, SEED_BASE + 3000)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    for view in (torch.int8, torch.uint8):
        a_d, b_d = ap.to(DEV).view(view), bp.to(DEV).view(view)
        c_d = poisoned_c(m, n, DEV)
        qm.gemm(a_d, b_d, c_d, m, n, k)
        assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1
        qm.gemm(a_d, b_d, c_d, m, n, k)  # twice into the same C: overwrite, not accumulate
        assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1


def test_k_zero_and_empty():
    c = poisoned_c(5, 7, DEV)
    e = torch.empty((5, 0), dtype=torch.int8, device=DEV)
    qm.gemm(e, torch.empty((7, 0), dtype=torch.int8, device=DEV), c, 5, 7, 0)
    assert (c == 0).all()
    qm.gemm(torch.empty((0, 16), dtype=torch.int8, device=DEV), torch.empty((7, 16), dtype=torch.int8, device=DEV),
            torch.empty((0, 7), dtype=torch.int32, device=DEV), 0, 7, 32)


def test_extension_module_runs_on_side_stream_and_under_graph_replay(oracle_mod):
    import quadmul

    m, n, k = 96, 160, 512
    a, b = make_operands(m, n, k, SEED_BASE + 3100)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    c_d = poisoned_c(m, n, DEV)
    quadmul.gemm(a_d, b_d, c_d, m, n, k)  # positional, as test.py:40
    torch.cuda.synchronize()
    assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1

    side = torch.cuda.Stream()
    c2 = poisoned_c(m, n, DEV)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        quadmul.gemm(a_d, b_d, c2, m, n, k)
    side.synchronize()
    assert oracle_mod.compare(c2.cpu().numpy(), want) == -1

    # captured as the reference's harness does (test.py:78-81); every replay is checked
    c3 = poisoned_c(m, n, DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(3):
            quadmul.gemm(a_d, b_d, c3, m, n, k)
    for _ in range(3):
        c3.fill_(0x7F7F7F7F)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert oracle_mod.compare(c3.cpu().numpy(), want) == -1


def test_dispatcher_op_eager_and_traced(oracle_mod):
    import quadmul  # noqa: F401

    m, n, k = 130, 200, 640
    a, b = make_operands(m, n, k, SEED_BASE + 3200)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    c_d = poisoned_c(m, n, DEV)
    torch.ops.quadmul.gemm(a_d, b_d, c_d, m, n, k)
    torch.cuda.synchronize()
    assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1

    def fn(x, y):
        out = torch.full((m, n), 0x7F7F7F7F, dtype=torch.int32, device=x.device)
        torch.ops.quadmul.gemm(x, y, out, m, n, k)
        return out

    traced = torch.compile(fn, backend="aot_eager", fullgraph=True)
    got = traced(a_d, b_d)
    torch.cuda.synchronize()
    assert oracle_mod.compare(got.cpu().numpy(), want) == -1


def test_pack_unpack_kernels(oracle_mod):
    from util import make_values

    for rows, k in [(1, 2), (3, 6), (7, 30), (16, 64), (33, 130), (128, 4096), (257, 1184)]:
        v = make_values(rows, k, SEED_BASE + 4000 + rows)
        want_p = oracle_mod.pack_i4(v.numpy())
        got_p = qm.pack_int4(v.to(DEV))
        assert (got_p.cpu().numpy().view(np.uint8) == want_p).all(), (rows, k)
        got_u = qm.unpack_int4(got_p)
        assert (got_u.cpu().numpy() == oracle_mod.unpack_i4(want_p)).all(), (rows, k)
        assert torch.equal(got_u.cpu(), v)
    allb = torch.arange(256, dtype=torch.uint8).view(4, 64).to(DEV)
    assert (qm.unpack_int4(allb).cpu().numpy() == oracle_mod.unpack_i4(allb.cpu().numpy())).all()
    assert torch.equal(qm.pack_int4(qm.unpack_int4(allb)).view(torch.uint8), allb)


# ------------------------------------------------------------------ the named workloads
NAMED_SHAPES = [
    (0, 1024, 1024, 1024), (1, 4096, 4096, 4096),
    (2, 1, 4096, 4096), (3, 16, 4096, 4096), (4, 64, 4096, 4096),
    (5, 2048, 11008, 4096), (6, 2048, 4096, 11008), (7, 2048, 12288, 4096),
]


@pytest.mark.parametrize("row", NAMED_SHAPES, ids=lambda r: "x".join(map(str, r[1:])))
def test_baseline_configs_full_compare(oracle_mod, row):
    i, m, n, k = row
    a, b = make_operands(m, n, k, SEED_BASE + i)
    ap, bp = pack_cpu(a), pack_cpu(b)
    got_d = poisoned_c(m, n, DEV)
    qm.gemm(ap.to(DEV), bp.to(DEV), got_d, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(got_d, fp32_matmul_on_gpu(a, b))
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy(), threads=0)
    assert oracle_mod.compare(got_d.cpu().numpy(), want) == -1


# More tiles than the device holds workgroups: every persistent workgroup runs several
# (K split, tile) items back to back, with 1, 2, 3 and 5 K-steps per item (the load
# cursor crosses item boundaries inside the ring; odd counts exercise the padding step),
# ragged edges, and the one-item-per-workgroup launch of the same configurations.
PERSISTENT_SHAPES = [(4352, 4400, 128), (4400, 4352, 256), (4352, 4400, 384), (2500, 9000, 640)]


@pytest.mark.parametrize("shape", PERSISTENT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_persistent_grid_many_items_per_workgroup(oracle_mod, shape):
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 5000 + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    want_d = fp32_matmul_on_gpu(a, b)
    rows = np.unique(np.concatenate([np.arange(0, m, 61), [m - 1, 255, 256, 257, 511, 512]])).astype(np.int32)
    want_rows = oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)
    assert oracle_mod.compare(want_d.cpu().numpy()[rows], want_rows) == -1  # the fast check agrees with the oracle
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("q") or not qm.config_supports(cfg, m, n, k):
            continue
        for gm, ks, spread in [(4, 1, 0), (1, 1, 0), (4, 1, 1), (3, 2, 0), (4, 3, 0), (2, 2, 1)]:
            got_d = poisoned_c(m, n, DEV)
            qm.gemm_cfg(a_d, b_d, got_d, m, n, k, cfg | (gm << 16) | (ks << 24) | (spread << 30))
            torch.cuda.synchronize()
            assert torch.equal(got_d, want_d), f"{name} group_m={gm} ksplit={ks} spread={spread}"
        ran += 1
    assert ran >= 4


def test_many_rounds_repeated(oracle_mod):
    """Many items per workgroup on every pipelined configuration, several times over: the
    write-out of one tile overlaps the loads of the next, so a misplaced wait shows up as an
    occasional wrong tile rather than every time (a three-stage ring once did exactly that)."""
    m, n, k = 2048, 28672, 256
    a, b = make_operands(m, n, k, SEED_BASE + 5100)
    ap, bp = pack_cpu(a), pack_cpu(b)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    want_d = fp32_matmul_on_gpu(a, b)
    rows = np.arange(0, m, 127).astype(np.int32)
    assert oracle_mod.compare(want_d.cpu().numpy()[rows], oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)) == -1
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("q"):
            continue
        for rep in range(6):
            got_d = poisoned_c(m, n, DEV)
            qm.gemm_cfg(a_d, b_d, got_d, m, n, k, cfg | ((1 + rep % 4) << 16))
            torch.cuda.synchronize()
            assert torch.equal(got_d, want_d), f"{name} repetition {rep}"


@pytest.mark.parametrize("row", [(8, 8192, 8192, 8192), (9, 8000, 8000, 8064)], ids=lambda r: "x".join(map(str, r[1:])))
def test_large_configs(oracle_mod, row):
    i, m, n, k = row
    a, b = make_operands(m, n, k, SEED_BASE + i)
    ap, bp = pack_cpu(a), pack_cpu(b)
    got_d = poisoned_c(m, n, DEV)
    qm.gemm(ap.to(DEV), bp.to(DEV), got_d, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(got_d, fp32_matmul_on_gpu(a, b))  # every element
    rows = np.unique(np.concatenate([np.arange(0, m, 97), [m - 1, m - 2, 255, 256, 257]])).astype(np.int32)
    want = oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)
    got = got_d.cpu().numpy()[rows]
    assert oracle_mod.compare(got, want) == -1
    # a checksum the layout cannot fake: column sums of C equal (sum of A rows) . B^T
    colsum = a.to(torch.int64).sum(0)
    want_cs = (b.to(torch.int64) * colsum).sum(1)
    assert torch.equal(got_d.to(torch.int64).sum(0).cpu(), want_cs)


@pytest.mark.parametrize("shape", [(128, 1024, 14336), (200, 300, 2048), (257, 511, 1280), (70, 4100, 4096)],
                         ids=lambda s: "x".join(map(str, s)))
def test_split_k_workspace_forms(oracle_mod, shape):
    """K split on the pipelined kernel: the caller's workspace in every form it can take --
    allocated by the wrapper, the caller's own tensor (exact size, larger, holding garbage),
    too small or absent (then atomics) -- gives the oracle's result."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 5200 + m)
    ap, bp = pack_cpu(a), pack_cpu(b)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("q") or not qm.config_supports(cfg, m, n, k):
            continue
        for gm, ks in [(1, 2), (3, 5), (8, 8)]:
            code = cfg | (gm << 16) | (ks << 24)
            need = qm.workspace_bytes(m, n, k, code)
            assert need > 0 and need % 16 == 0
            garbage = torch.randint(-128, 128, (need + 4096,), dtype=torch.int8, device=DEV).view(torch.uint8)
            for what, ws in [("wrapper", True), ("exact", garbage[:need]), ("larger", garbage), ("too small", garbage[:need - 16]),
                             ("none", None)]:
                c_d = poisoned_c(m, n, DEV)
                qm.gemm_cfg(a_d, b_d, c_d, m, n, k, code, ws)
                torch.cuda.synchronize()
                bad = oracle_mod.compare(c_d.cpu().numpy(), want)
                assert bad == -1, f"{name} group_m={gm} ksplit={ks} workspace {what}: first mismatch at flat index {bad}"
        ran += 1
    assert ran >= 4


def test_auto_choice_splits_k_and_matches(oracle_mod):
    # few tiles, long K: the automatic choice splits K; extension module and wrapper agree with the oracle
    import quadmul

    m, n, k = 450, 1280, 28672
    code = qm.select_config(m, n, k)
    assert qm.config_name(code & 0xFFFF).startswith("q") and (code >> 24) & 0x3F > 1
    assert qm.workspace_bytes(m, n, k) > 0
    a, b = make_operands(m, n, k, SEED_BASE + 5300)
    ap, bp = pack_cpu(a), pack_cpu(b)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    for fn in (lambda c: quadmul.gemm(a_d, b_d, c, m, n, k), lambda c: qm.gemm(a_d, b_d, c, m, n, k),
               lambda c: qm.gemm(a_d, b_d, c, m, n, k, workspace=None), lambda c: torch.ops.quadmul.gemm(a_d, b_d, c, m, n, k)):
        c_d = poisoned_c(m, n, DEV)
        fn(c_d)
        torch.cuda.synchronize()
        assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1
    # captured in a graph (the workspace comes from the allocator's graph pool) and replayed
    c_d = poisoned_c(m, n, DEV)
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        quadmul.gemm(a_d, b_d, c_d, m, n, k)
        with torch.cuda.graph(g, stream=side):
            quadmul.gemm(a_d, b_d, c_d, m, n, k)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        c_d.fill_(C_POISON)
        g.replay()
        torch.cuda.synchronize()
        assert oracle_mod.compare(c_d.cpu().numpy(), want) == -1


def test_random_shapes_through_the_automatic_choice():
    """A seeded sweep of shapes nobody tuned for, through qm_gemm_i4's own choice of kernel
    (table, cost model, K split with a workspace, generic fallback), against an fp32 matmul
    on the GPU (exact: every partial sum is an integer below 2^24)."""
    import quadmul

    rng = np.random.default_rng(SEED_BASE + 5400)
    seen = set()
    for i in range(160):
        m = int(np.exp(rng.uniform(0, np.log(1500)))) if i % 3 else int(rng.integers(1, 140))
        n = int(np.exp(rng.uniform(0, np.log(6000))))
        kind = i % 4
        k = int(np.exp(rng.uniform(np.log(2), np.log(12000))))
        k = max(2, [k // 128 * 128, k // 32 * 32, k // 2 * 2, k // 128 * 128][kind])
        if i % 10 == 0:
            m, k = int(rng.integers(65, 129)), int(rng.integers(8, 64)) * 128   # the 128-row skinny kernel
        if i % 10 == 5:   # few tiles, long K: the pipelined kernel with K split through a workspace
            m, n, k = int(rng.integers(450, 1000)), int(rng.integers(1100, 1500)), int(rng.integers(224, 257)) * 128
        if i % 10 == 7:   # many tiles: the pipelined kernel, persistent grid
            m, n, k = int(rng.integers(700, 1500)), int(rng.integers(3000, 6000)), int(rng.integers(4, 16)) * 128
        a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=torch.Generator().manual_seed(1000 + i))
        b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=torch.Generator().manual_seed(2000 + i))
        a_d, b_d = pack_cpu(a).to(DEV), pack_cpu(b).to(DEV)
        want = fp32_matmul_on_gpu(a, b)
        c_d = poisoned_c(m, n, DEV)
        quadmul.gemm(a_d, b_d, c_d, m, n, k)
        torch.cuda.synchronize()
        code = qm.select_config(m, n, k)
        name = qm.config_name(code & 0xFFFF)
        seen.add(name[0] + ("+split" if (code >> 24) & 0x3F > 1 else ""))
        assert torch.equal(c_d, want), f"{m}x{n}x{k} ({name}, ksplit {(code >> 24) & 0x3F})"
        # nothing of 2^27 multiply-adds or more is left to the one-thread-per-element kernel:
        # where no fast kernel takes the operands as they are, the call runs on padded copies
        # in the workspace (which quadmul.gemm provides)
        if name == "generic" and m * n * ((k + 127) // 128 * 128) >= 2 ** 27 and k <= 131000:
            assert qm.workspace_bytes(m, n, k) > 0, (m, n, k)
    assert {"g", "d", "p", "q", "q+split"} <= seen, seen


@pytest.mark.parametrize("shape", [(1, 4096, 4096), (2, 4100, 11008), (1, 50, 131040), (2, 33, 28672), (1, 4096, 96)],
                         ids=lambda s: "x".join(map(str, s)))
def test_dot_product_kernel_one_and_two_rows(oracle_mod, shape):
    """The GEMV-like kernel (v_dot8_i32_i4 on the packed nibbles as they are): random data
    against the oracle, the extremes in closed form, on every such configuration."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 5500 + n)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    lo_a = pack_cpu(torch.full((m, k), -8, dtype=torch.int8))
    lo_b, hi_b = pack_cpu(torch.full((n, k), -8, dtype=torch.int8)), pack_cpu(torch.full((n, k), 7, dtype=torch.int8))
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("v") or not qm.config_supports(cfg, m, n, k):
            continue
        assert oracle_mod.compare(run_gemm(ap, bp, m, n, k, cfg), want) == -1, name
        assert (run_gemm(lo_a, lo_b, m, n, k, cfg) == 64 * k).all(), name
        assert (run_gemm(lo_a, hi_b, m, n, k, cfg) == -56 * k).all(), name
        ran += 1
    assert ran >= (2 if m == 1 else 1)
    assert qm.config_name(qm.select_config(m, n, k) & 0xFFFF).startswith("v")
    assert oracle_mod.compare(run_gemm(ap, bp, m, n, k), want) == -1


@pytest.mark.parametrize("shape", [(3000, 3000, 1056), (1000, 1000, 1000), (1000, 1100, 1004), (300, 5000, 4098), (2100, 4200, 96 + 2),
                                   (2100, 4200, 96), (1500, 1500, 64), (4096, 4096, 32)],
                         ids=lambda s: "x".join(map(str, s)))
def test_k_padded_through_the_workspace(shape):
    """Large shapes whose K is not a multiple of 32, and unaligned operands: with a workspace
    the operands are copied with zero-padded rows and the pipelined kernel runs; without one
    the generic kernel does.  (K % 32 == 0, first case: no copies, a short last K-step; a K of
    less than one K-step: no copies either, 32 x 32 blocks of the wave-level kernel.)  Same
    result, against an exact fp32 matmul."""
    import quadmul

    m, n, k = shape
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=torch.Generator().manual_seed(SEED_BASE + 5600 + k))
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=torch.Generator().manual_seed(SEED_BASE + 5700 + k))
    want = fp32_matmul_on_gpu(a, b)
    ap, bp = pack_cpu(a), pack_cpu(b)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    if k % 32:
        assert qm.workspace_bytes(m, n, k) >= (m + n) * ((k + 127) // 128 * 64)
    elif k < 128:   # (less than one whole K-step: nothing for a short last step to follow)
        assert qm.workspace_bytes(m, n, k) == 0 and qm.config_name(qm.select_config(m, n, k) & 0xFFFF).startswith("d2x2")
    else:   # K % 32 == 0: the pipelined kernel runs it as it is, with a short last K-step
        assert qm.workspace_bytes(m, n, k) == 0 and qm.config_name(qm.select_config(m, n, k) & 0xFFFF).startswith("q")
    for fn in (lambda c: quadmul.gemm(a_d, b_d, c, m, n, k), lambda c: qm.gemm(a_d, b_d, c, m, n, k),
               lambda c: qm.gemm(a_d, b_d, c, m, n, k, workspace=None),
               lambda c: qm.gemm(a_d, b_d, c, m, n, k, workspace=torch.empty(4096, dtype=torch.uint8, device=DEV))):
        c_d = poisoned_c(m, n, DEV)
        fn(c_d)
        torch.cuda.synchronize()
        assert torch.equal(c_d, want)
    # operands at odd addresses
    a_buf = torch.empty(ap.numel() + 1, dtype=torch.int8, device=DEV)
    b_buf = torch.empty(bp.numel() + 3, dtype=torch.int8, device=DEV)
    a_odd, b_odd = a_buf[1:].view(m, k // 2), b_buf[3:].view(n, k // 2)
    a_odd.copy_(a_d)
    b_odd.copy_(b_d)
    assert a_odd.data_ptr() % 2 == 1
    c_d = poisoned_c(m, n, DEV)
    qm.gemm(a_odd, b_odd, c_d, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(c_d, want)


@pytest.mark.parametrize("k", [160, 192, 224, 288, 4128, 4160, 4192, 11040], ids=lambda k: f"k{k}")
def test_short_last_k_step_on_every_pipelined_config(oracle_mod, k):
    """K % 128 = 32, 64, 96: the last K-step of the pipelined kernel is loaded as the last 128
    nibbles of the row and the overlap with the step before is masked; whole and ragged tiles,
    K splits (the split that holds the short step keeps two steps), both item orders."""
    m, n = 300, 520
    a, b = make_operands(m, n, k, SEED_BASE + 5800 + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    hi_a, lo_b = pack_cpu(torch.full((m, k), 7, dtype=torch.int8)), pack_cpu(torch.full((n, k), -8, dtype=torch.int8))
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("q"):
            continue
        assert qm.config_supports(cfg, m, n, k), name
        for gm, ks, spread in [(1, 1, 0), (4, 1, 1), (2, 2, 0), (3, 3, 0), (1, 16, 0)]:
            code = cfg | (gm << 16) | (ks << 24) | (spread << 30)
            for ws in ([True, None] if ks > 1 else [True]):
                got = run_gemm(ap, bp, m, n, k, code, ws)
                bad = oracle_mod.compare(got, want)
                assert bad == -1, f"{name} group_m={gm} ksplit={ks} spread={spread} workspace={ws}: first mismatch at flat index {bad}"
        assert (run_gemm(hi_a, lo_b, m, n, k, cfg) == -56 * k).all(), name   # every nibble counted exactly once
        ran += 1
    assert ran >= 8


def test_operands_of_two_gib_and_more(oracle_mod):
    """An A of 2 GiB or more is cut into row blocks that fit the fast kernels' 32-bit row
    offsets, a B that large into blocks of its rows (blocks of columns of C, written through a
    row stride).  Every row is compared
    with the library's own result on slices below the limit (paths the other tests pin against
    the oracle), and the rows either side of the block boundary and the last rows with the
    oracle itself.  Packed bytes are drawn on the GPU: any byte is two valid nibbles."""
    import quadmul

    k, kb = 4096, 2048
    g = torch.Generator(device=DEV).manual_seed(SEED_BASE + 6100)
    # --- large A ---
    m, n = (1 << 20) + 300, 48
    assert m * kb >= 2 ** 31
    a_d = torch.randint(-128, 128, (m, kb), dtype=torch.int8, device=DEV, generator=g)
    b_d = torch.randint(-128, 128, (n, kb), dtype=torch.int8, device=DEV, generator=g)
    want = torch.empty((m, n), dtype=torch.int32, device=DEV)
    for r0 in range(0, m, 65536):
        rows = min(65536, m - r0)
        qm.gemm(a_d[r0:r0 + rows], b_d, want[r0:r0 + rows], rows, n, k)
    block = ((2 ** 31 - 2) // kb) & ~255
    assert 0 < block < m
    for fn in (lambda c: quadmul.gemm(a_d, b_d, c, m, n, k), lambda c: qm.gemm(a_d, b_d, c, m, n, k, workspace=None)):
        c_d = poisoned_c(m, n, DEV)
        fn(c_d)
        torch.cuda.synchronize()
        assert torch.equal(c_d, want)
    for r0 in (0, block - 24, m - 40):
        ref = oracle_mod.gemm_i4(a_d[r0:r0 + 40].cpu().numpy(), b_d.cpu().numpy())
        assert oracle_mod.compare(c_d[r0:r0 + 40].cpu().numpy(), ref) == -1
    # the scaled output takes the same road, with the row scales of each block
    rs = torch.rand(m, device=DEV, generator=g) * 0.01 + 0.001
    cs = torch.rand(n, device=DEV, generator=g) + 0.5
    d_d = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
    torch.cuda.synchronize()
    for r0 in (0, block - 24, m - 40):
        ref = oracle_mod.scale_round16(want[r0:r0 + 40].cpu().numpy(), rs[r0:r0 + 40].cpu().numpy(), cs.cpu().numpy(), oracle_mod.OUT_F16)
        assert np.array_equal(d_d[r0:r0 + 40].cpu().numpy().view(np.uint16), ref)
    del a_d, want, c_d, d_d
    # --- large B: cut into blocks of its rows, i.e. blocks of columns of C, which the kernels
    # write through a row stride; a skinny shape and one for the pipelined tile kernel ---
    n = (1 << 20) + 20
    assert n * kb >= 2 ** 31
    b_d = torch.randint(-128, 128, (n, kb), dtype=torch.int8, device=DEV, generator=g)
    block = ((2 ** 31 - 2) // kb) & ~255
    assert 0 < block < n
    for m in (8, 300):
        a_d = torch.randint(-128, 128, (m, kb), dtype=torch.int8, device=DEV, generator=g)
        assert qm.workspace_bytes(m, n, k) == 0
        c_d = poisoned_c(m, n, DEV)
        quadmul.gemm(a_d, b_d, c_d, m, n, k)
        torch.cuda.synchronize()
        for c0 in range(0, n, 262144):
            cols = min(262144, n - c0)
            part = torch.empty((m, cols), dtype=torch.int32, device=DEV)
            qm.gemm(a_d, b_d[c0:c0 + cols], part, m, cols, k)
            assert torch.equal(c_d[:, c0:c0 + cols], part), (m, c0)
        for c0 in (0, block - 30, n - 50):
            ref = oracle_mod.gemm_i4(a_d.cpu().numpy(), b_d[c0:c0 + 50].cpu().numpy())
            assert oracle_mod.compare(np.ascontiguousarray(c_d[:, c0:c0 + 50].cpu().numpy()), ref) == -1
        # the scaled output: column scales follow the blocks
        rs = torch.rand(m, device=DEV, generator=g) * 0.01 + 0.001
        cs = torch.rand(n, device=DEV, generator=g) + 0.5
        d_d = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
        quadmul.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
        torch.cuda.synchronize()
        for c0 in (0, block - 30, n - 50):
            ref = oracle_mod.scale_round16(np.ascontiguousarray(c_d[:, c0:c0 + 50].cpu().numpy()), rs.cpu().numpy(), cs[c0:c0 + 50].cpu().numpy(),
                                           oracle_mod.OUT_BF16)
            assert np.array_equal(np.ascontiguousarray(d_d[:, c0:c0 + 50].view(torch.int16).cpu().numpy()).view(np.uint16), ref), (m, c0)
        del a_d, c_d, d_d


def test_host_threads_on_their_own_streams():
    """Four host threads, each with its own stream, operands, output and workspace, call the
    library at the same time (ctypes drops the GIL for the call): shapes for the pipelined
    kernel, a K split through the workspace, the skinny and the dot kernel.  Every result of
    every round equals the one computed alone beforehand."""
    import threading

    shapes = [(512, 768, 2048), (256, 256, 65536), (16, 4096, 4096), (1, 2048, 8192)]
    jobs = []
    for i, (m, n, k) in enumerate(shapes):
        g = torch.Generator(device=DEV).manual_seed(SEED_BASE + 6300 + i)
        a_d = torch.randint(-128, 128, (m, k // 2), dtype=torch.int8, device=DEV, generator=g)
        b_d = torch.randint(-128, 128, (n, k // 2), dtype=torch.int8, device=DEV, generator=g)
        want = torch.empty((m, n), dtype=torch.int32, device=DEV)
        qm.gemm(a_d, b_d, want, m, n, k)
        ws = torch.empty(max(qm.workspace_bytes(m, n, k), 16), dtype=torch.uint8, device=DEV)
        jobs.append((m, n, k, a_d, b_d, want, ws))
    torch.cuda.synchronize()
    assert qm.workspace_bytes(*shapes[1]) > 0
    failures = []

    def worker(job):
        m, n, k, a_d, b_d, want, ws = job
        stream = torch.cuda.Stream(device=DEV)
        try:
            with torch.cuda.stream(stream):
                for _ in range(40):
                    c_d = poisoned_c(m, n, DEV)
                    qm.gemm(a_d, b_d, c_d, m, n, k, workspace=ws)
                    if not torch.equal(c_d, want):
                        failures.append((m, n, k))
                        return
            stream.synchronize()
        except Exception as ex:  # a thread's exception would otherwise be lost
            failures.append((m, n, k, repr(ex)))

    threads = [threading.Thread(target=worker, args=(job,)) for job in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert failures == []


@pytest.mark.parametrize("shape", [(16, 11008, 4096), (3, 8210, 1024), (128, 8195, 1056), (40, 16400, 2048), (1, 24577, 512)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_kernel_walking_over_column_blocks(oracle_mod, shape):
    """More column blocks than two workgroups per CU hold at once and K within one turn of the
    waves: the skinny kernel's workgroups walk over several blocks each, A fragments kept,
    B of the next block prefetched, sums in alternating halves of the LDS.  Every skinny
    configuration that takes the shape, int32 and scaled output, against the oracle."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 6500 + n)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    g = torch.Generator().manual_seed(SEED_BASE + 6600 + n)
    rs, cs = torch.rand(m, generator=g) * 0.01 + 0.001, torch.rand(n, generator=g) + 0.5
    want16 = oracle_mod.scale_round16(want, rs.numpy(), cs.numpy(), oracle_mod.OUT_BF16)
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("s") or not qm.config_supports(cfg, m, n, k):
            continue
        c_d = poisoned_c(m, n, DEV)
        qm.gemm_cfg(a_d, b_d, c_d, m, n, k, cfg)
        d_d = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
        qm.gemm_scaled(a_d, b_d, d_d, m, n, k, rs.to(DEV), cs.to(DEV), cfg)
        torch.cuda.synchronize()
        bad = oracle_mod.compare(c_d.cpu().numpy(), want)
        assert bad == -1, f"{name}: first mismatch at flat index {bad}"
        assert np.array_equal(d_d.view(torch.int16).cpu().numpy().view(np.uint16), want16), name
        ran += 1
    assert ran >= 2


@pytest.mark.parametrize("shape", [(16, 9000, 4096), (3, 8210, 1024 + 32), (30, 4100, 2048 + 96), (13, 5000, 8192), (16, 300, 14336 + 64),
                                   (50, 4200, 4096 + 32), (7, 33, 32), (16, 16, 65536),
                                   # several blocks of rows (the "d" form's grid walks over them), the last one ragged
                                   (64, 4096, 4096), (100, 4200, 4096 + 32), (200, 1000, 2048 + 64), (129, 530, 8192), (33, 8300, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_kernels_streaming_global_to_lds(oracle_mod, shape):
    """The skinny kernels whose operands go global -> LDS directly ("d": one workgroup per
    block of rows and of columns, a ring of runs per wave refilled over a long K; "p": a persistent grid
    walking over more column blocks than the device holds workgroups, A resident in
    registers): ragged N, short last runs of K (K % 256 = 32, 64, 96), K from one run to 256
    runs per row.  Every such configuration that takes the shape, int32 and scaled output,
    against the oracle; the extremes in closed form."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 6700 + n + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    g = torch.Generator().manual_seed(SEED_BASE + 6800 + n)
    rs, cs = torch.rand(m, generator=g) * 0.01 + 0.001, torch.rand(n, generator=g) + 0.5
    want16 = oracle_mod.scale_round16(want, rs.numpy(), cs.numpy(), oracle_mod.OUT_F16)
    lo_a = pack_cpu(torch.full((m, k), -8, dtype=torch.int8))
    lo_b, hi_b = pack_cpu(torch.full((n, k), -8, dtype=torch.int8)), pack_cpu(torch.full((n, k), 7, dtype=torch.int8))
    ran = set()
    for cfg, name in enumerate(qm.config_names()):
        if name[0] not in "dp" or not qm.config_supports(cfg, m, n, k):
            continue
        c_d = poisoned_c(m, n, DEV)
        qm.gemm_cfg(a_d, b_d, c_d, m, n, k, cfg)
        d_d = torch.zeros((m, n), dtype=torch.float16, device=DEV)
        qm.gemm_scaled(a_d, b_d, d_d, m, n, k, rs.to(DEV), cs.to(DEV), cfg)
        torch.cuda.synchronize()
        bad = oracle_mod.compare(c_d.cpu().numpy(), want)
        assert bad == -1, f"{name}: first mismatch at flat index {bad}"
        assert np.array_equal(d_d.view(torch.int16).cpu().numpy().view(np.uint16), want16), name
        if k <= 28672:
            assert (run_gemm(lo_a, lo_b, m, n, k, cfg) == 64 * k).all(), name
            assert (run_gemm(lo_a, hi_b, m, n, k, cfg) == -56 * k).all(), name
        ran.add(name[0])
    assert "d" in ran and (k > 8192 or m > 32 or "p" in ran), ran
    if m > 2:
        assert qm.config_name(qm.select_config(m, n, k) & 0xFFFF)[0] in "dp"


def test_every_config_on_random_shapes_against_the_generic_kernel():
    """A bounded soak: every configuration on random shapes it supports, ragged in all three
    dimensions, with and without a K split, against the generic kernel on the same operands
    (one thread per element, itself checked against the oracle above)."""
    rng = np.random.default_rng(SEED_BASE + 77)
    names = qm.config_names()
    generic = names.index("generic")
    skinny_m = [1, 2, 3, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 129, 200]
    skinny_n = [1, 5, 16, 17, 100, 255, 256, 1000, 4096, 4100, 9000]
    skinny_k = [1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 32, 33, 64, 100, 127, 128, 129, 256, 300]
    tile_m = [1, 16, 63, 64, 65, 128, 200, 256, 257, 512, 700]
    tile_n = [8, 64, 100, 128, 256, 260, 512, 1000, 1300]
    tile_k = [1, 2, 3, 4, 5, 8, 12, 13, 16, 31, 32, 40, 64, 65]
    ran = {}
    gen = torch.Generator(device=DEV)
    for it in range(20000):
        cfg = int(rng.integers(len(names)))
        if cfg == generic:
            continue
        tile = names[cfg][0] == "q"
        m = int(rng.choice(tile_m if tile else skinny_m))
        n = int(rng.choice(tile_n if tile else skinny_n))
        k = 32 * int(rng.choice(tile_k if tile else skinny_k))
        if not qm.config_supports(cfg, m, n, k):
            continue
        seed = SEED_BASE + 770000 + it   # of this case's operands: a failure can be replayed alone
        gen.manual_seed(seed)
        a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=DEV, generator=gen)
        b = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=DEV, generator=gen)
        want = poisoned_c(m, n, DEV)
        qm.gemm_cfg(a, b, want, m, n, k, generic)
        ksplit = int(rng.choice([1, 1, 2, 3])) if tile and k >= 256 else 1
        got = poisoned_c(m, n, DEV)
        qm.gemm_cfg(a, b, got, m, n, k, cfg | (ksplit << 24) if ksplit > 1 else cfg, workspace=True if rng.integers(2) else None)
        assert torch.equal(want, got), (names[cfg], ksplit, m, n, k, f"operand seed {seed}")
        ran[names[cfg]] = ran.get(names[cfg], 0) + 1
    assert len(ran) == len(names) - 1 and min(ran.values()) >= 10, ran
