"""GPU parity of the GEMM with the fused dequantising epilogue (scaled fp16 / bf16 output),
called through the C ABI, against the CPU oracle -- bit-exact on the 16-bit patterns."""
import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import SEED_BASE, make_operands, pack_cpu

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [(torch.float16, 1), (torch.bfloat16, 2)]


def make_scales(m, n, seed):
    g = torch.Generator().manual_seed(seed)
    rs = torch.rand(m, generator=g) * 0.02 + 1e-3   # per-token activation scales
    cs = torch.rand(n, generator=g) * 0.05 + 1e-4   # per-channel weight scales
    return rs.float(), cs.float()


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def poisoned_d(m, n, dtype):
    return torch.full((m, n), float("nan"), dtype=dtype, device=DEV)


SHAPES = [(1, 1, 128), (15, 17, 128), (17, 63, 256), (65, 255, 384), (128, 256, 4096), (200, 300, 1152), (257, 511, 256),
          (300, 70, 2048), (3, 5, 30), (70, 33, 162), (64, 64, 96)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_every_scaled_config_matches_oracle(oracle_mod, shape):
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 7000 + m + 3 * n + k)
    ap, bp = pack_cpu(a), pack_cpu(b)
    rs, cs = make_scales(m, n, SEED_BASE + 7100 + m)
    c = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d, rs_d, cs_d = ap.to(DEV), bp.to(DEV), rs.to(DEV), cs.to(DEV)
    ran = 0
    for dtype, out in DTYPES:
        want = oracle_mod.scale_round16(c, rs.numpy(), cs.numpy(), out)
        for cfg, name in enumerate(qm.config_names()):
            if not (qm.config_has_scaled(cfg) and qm.config_supports(cfg, m, n, k)):
                continue
            for gm, spread in [(1, 0), (3, 1)]:
                d = poisoned_d(m, n, dtype)
                qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d, cfg | (gm << 16) | (spread << 30))
                torch.cuda.synchronize()
                got = bits(d)
                bad = np.flatnonzero(got != want)
                assert bad.size == 0, f"{name} {dtype} group_m={gm}: {bad.size} mismatches, first at {bad[0]}: got {got.flat[bad[0]]:#06x} want {want.flat[bad[0]]:#06x}"
            ran += 1
        d = poisoned_d(m, n, dtype)
        qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d)
        torch.cuda.synchronize()
        assert (bits(d) == want).all()
    assert ran >= 2


def test_missing_scales_and_k_zero(oracle_mod):
    m, n, k = 130, 260, 512
    a, b = make_operands(m, n, k, SEED_BASE + 7200)
    ap, bp = pack_cpu(a), pack_cpu(b)
    c = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    rs, cs = make_scales(m, n, SEED_BASE + 7201)
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    for dtype, out in DTYPES:
        for r_, c_ in [(None, None), (rs, None), (None, cs)]:
            d = poisoned_d(m, n, dtype)
            qm.gemm_scaled(a_d, b_d, d, m, n, k, None if r_ is None else r_.to(DEV), None if c_ is None else c_.to(DEV))
            torch.cuda.synchronize()
            want = oracle_mod.scale_round16(c, None if r_ is None else r_.numpy(), None if c_ is None else c_.numpy(), out)
            assert (bits(d) == want).all()
        d = poisoned_d(5, 7, dtype)
        e = torch.empty((5, 0), dtype=torch.int8, device=DEV)
        qm.gemm_scaled(e, torch.empty((7, 0), dtype=torch.int8, device=DEV), d, 5, 7, 0)
        torch.cuda.synchronize()
        assert (bits(d) == 0).all()


def test_rejections():
    m, n, k = 64, 64, 512
    a = torch.zeros((m, k // 2), dtype=torch.int8, device=DEV)
    d = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    names = qm.config_names()
    with pytest.raises(qm.QuadmulError):  # the 256 x 128 tile two to a CU has no scaled output (its registers do not hold the scales)
        qm.gemm_scaled(a, a, d, m, n, k, None, None, names.index("q256x128_w2x2_s3o2"))
    with pytest.raises(qm.QuadmulError):  # partial sums cannot meet in a rounded output: a K split needs a workspace
        qm.gemm_scaled(a, a, d, m, n, k, None, None, names.index("q128x128_w2x2_s7o1") | (2 << 24), workspace=None)
    with pytest.raises(qm.QuadmulError):
        qm.gemm_scaled(a, a, d, m, n, k, None, None, names.index("q128x128_w2x2_s7o1") | (2 << 24),
                       workspace=torch.empty(1024, dtype=torch.uint8, device=DEV))
    with pytest.raises(qm.QuadmulError):  # only the pipelined kernel splits K
        qm.gemm_scaled(a, a, d, m, n, k, None, None, names.index("s4x1_w8_u2") | (2 << 24))
    with pytest.raises(qm.QuadmulError):
        qm.gemm_scaled(a, a, torch.zeros((m, n), dtype=torch.int32, device=DEV), m, n, k)
    with pytest.raises(qm.QuadmulError):
        qm.gemm_scaled(a, a, d, m, n, k, torch.ones(m, dtype=torch.float16, device=DEV))
    lib = qm.library()
    assert lib.qm_gemm_i4_scaled(a.data_ptr(), a.data_ptr(), d.data_ptr(), m, n, k, None, None, 3, None) == -6
    assert lib.qm_gemm_i4_scaled(a.data_ptr(), a.data_ptr(), d.data_ptr() + 1, m, n, k, None, None, 1, None) == -5


BIG = [(4096, 4096, 4096), (2048, 11008, 4096), (16, 4096, 4096), (8000, 4200, 1024), (512, 6144, 4096), (100, 4096, 200)]


@pytest.mark.parametrize("shape", BIG, ids=lambda s: "x".join(map(str, s)))
def test_scaled_large_shapes_every_element(oracle_mod, shape):
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 7300 + m)
    ap, bp = pack_cpu(a), pack_cpu(b)
    rs, cs = make_scales(m, n, SEED_BASE + 7301)
    a_d, b_d, rs_d, cs_d = ap.to(DEV), bp.to(DEV), rs.to(DEV), cs.to(DEV)
    c_d = torch.empty((m, n), dtype=torch.int32, device=DEV)
    qm.gemm(a_d, b_d, c_d, m, n, k)  # the int32 path has its own parity tests
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 23)), [m - 1]])).astype(np.int32)
    c_rows = oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)
    assert (c_d.cpu().numpy()[rows] == c_rows).all()
    for dtype, out in DTYPES:
        d = poisoned_d(m, n, dtype)
        qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d)
        torch.cuda.synchronize()
        # every element: the same two float32 multiplications and the same rounding, by torch on the GPU
        want_d = ((c_d.to(torch.float32) * rs_d[:, None]) * cs_d[None, :]).to(dtype)
        assert torch.equal(d.view(torch.int16), want_d.view(torch.int16))
        # sampled rows against the oracle
        want = oracle_mod.scale_round16(c_rows, rs.numpy()[rows], cs.numpy(), out)
        assert (bits(d)[rows] == want).all()


def test_extension_module_and_dispatcher_op(oracle_mod):
    import quadmul

    m, n, k = 200, 264, 640
    a, b = make_operands(m, n, k, SEED_BASE + 7400)
    ap, bp = pack_cpu(a), pack_cpu(b)
    rs, cs = make_scales(m, n, SEED_BASE + 7401)
    c = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d, rs_d, cs_d = ap.to(DEV), bp.to(DEV), rs.to(DEV), cs.to(DEV)
    for dtype, out in DTYPES:
        want = oracle_mod.scale_round16(c, rs.numpy(), cs.numpy(), out)
        d = poisoned_d(m, n, dtype)
        quadmul.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d)
        torch.cuda.synchronize()
        assert (bits(d) == want).all()
        d2 = poisoned_d(m, n, dtype)
        torch.ops.quadmul.gemm_scaled(a_d, b_d, d2, m, n, k, rs_d, cs_d)

        def fn(x, y, r, s_):
            o = torch.full((m, n), float("nan"), dtype=dtype, device=x.device)
            torch.ops.quadmul.gemm_scaled(x, y, o, m, n, k, r, s_)
            return o

        d3 = torch.compile(fn, backend="aot_eager", fullgraph=True)(a_d, b_d, rs_d, cs_d)
        torch.cuda.synchronize()
        assert (bits(d2) == want).all() and (bits(d3) == want).all()
        # captured and replayed, every replay checked
        d4 = poisoned_d(m, n, dtype)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            quadmul.gemm_scaled(a_d, b_d, d4, m, n, k, rs_d, cs_d)
        for _ in range(3):
            d4.fill_(float("nan"))
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert (bits(d4) == want).all()
    with pytest.raises(RuntimeError):
        quadmul.gemm_scaled(a_d, b_d, torch.zeros((m, n), dtype=torch.float32, device=DEV), m, n, k)


@pytest.mark.parametrize("shape", [(128, 1024, 14336), (200, 300, 2048), (257, 511, 1280)], ids=lambda s: "x".join(map(str, s)))
def test_scaled_with_k_split_through_a_workspace(oracle_mod, shape):
    """With a workspace the scaled form takes K splits on every pipelined configuration: the
    int32 partial tiles are added up, scaled and rounded by the second kernel."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 7300 + m)
    ap, bp = pack_cpu(a), pack_cpu(b)
    rs, cs = make_scales(m, n, SEED_BASE + 7400 + m)
    c = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d, rs_d, cs_d = ap.to(DEV), bp.to(DEV), rs.to(DEV), cs.to(DEV)
    ran = 0
    for dtype, out in DTYPES:
        want = oracle_mod.scale_round16(c, rs.numpy(), cs.numpy(), out)
        want_rows_only = oracle_mod.scale_round16(c, rs.numpy(), None, out)
        for cfg, name in enumerate(qm.config_names()):
            if not name.startswith("q") or not qm.config_supports(cfg, m, n, k):
                continue
            for gm, ks in [(1, 2), (3, 5)]:
                code = cfg | (gm << 16) | (ks << 24)
                assert qm.workspace_bytes(m, n, k, code, scaled=True) > 0
                d = poisoned_d(m, n, dtype)
                qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d, code)
                torch.cuda.synchronize()
                got = bits(d)
                bad = np.flatnonzero(got != want)
                assert bad.size == 0, f"{name} {dtype} group_m={gm} ksplit={ks}: {bad.size} mismatches, first at {bad[0]}"
            d = poisoned_d(m, n, dtype)
            qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, None, cfg | (4 << 24))
            torch.cuda.synchronize()
            assert (bits(d) == want_rows_only).all(), name
            ran += 1
    assert ran >= 8


def test_scaled_random_shapes_through_the_automatic_choice():
    """The same sweep for the scaled output, against torch's float32 arithmetic on the exact
    int32 product (two separate float32 multiplications, then torch's rounding to 16 bits)."""
    rng = np.random.default_rng(SEED_BASE + 7500)
    for i in range(80):
        m = int(np.exp(rng.uniform(0, np.log(1200)))) if i % 3 else int(rng.integers(1, 140))
        n = int(np.exp(rng.uniform(0, np.log(5000))))
        k = int(np.exp(rng.uniform(np.log(2), np.log(12000))))
        k = max(2, [k // 128 * 128, k // 32 * 32, k // 2 * 2, k // 128 * 128][i % 4])
        if i % 8 == 0:
            m, k = int(rng.integers(65, 129)), int(rng.integers(16, 96)) * 128
        a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=torch.Generator().manual_seed(3000 + i))
        b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=torch.Generator().manual_seed(4000 + i))
        rs, cs = make_scales(m, n, 5000 + i)
        a_d, b_d, rs_d, cs_d = pack_cpu(a).to(DEV), pack_cpu(b).to(DEV), rs.to(DEV), cs.to(DEV)
        c32 = (a.to(DEV).float() @ b.to(DEV).float().t())   # exact integers in fp32
        dtype = torch.float16 if i % 2 else torch.bfloat16
        want = ((c32 * rs_d[:, None]) * cs_d[None, :]).to(dtype)
        d = poisoned_d(m, n, dtype)
        qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d)
        torch.cuda.synchronize()
        assert torch.equal(d.view(torch.int16), want.view(torch.int16)), f"{m}x{n}x{k} {dtype}"


def test_scaled_k_padded_through_the_workspace():
    m, n, k = 3000, 3000, 1058
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=torch.Generator().manual_seed(SEED_BASE + 7600))
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=torch.Generator().manual_seed(SEED_BASE + 7700))
    rs, cs = make_scales(m, n, SEED_BASE + 7800)
    a_d, b_d, rs_d, cs_d = pack_cpu(a).to(DEV), pack_cpu(b).to(DEV), rs.to(DEV), cs.to(DEV)
    c32 = a.to(DEV).float() @ b.to(DEV).float().t()
    assert qm.workspace_bytes(m, n, k, scaled=True) > 0
    for dtype in (torch.float16, torch.bfloat16):
        want = ((c32 * rs_d[:, None]) * cs_d[None, :]).to(dtype)
        for ws in (True, None):
            d = poisoned_d(m, n, dtype)
            qm.gemm_scaled(a_d, b_d, d, m, n, k, rs_d, cs_d, workspace=ws)
            torch.cuda.synchronize()
            assert torch.equal(d.view(torch.int16), want.view(torch.int16)), (dtype, ws)


@pytest.mark.parametrize("shape", [(700, 1300, 512), (1290, 520, 384), (2100, 2052, 256 + 32), (300, 4100, 1024)], ids=lambda s: "x".join(map(str, s)))
def test_tiles_that_stick_out_of_c_on_every_pipelined_configuration(oracle_mod, shape):
    """N % 4 == 0 and an aligned C: whole tiles and tiles that stick out of the matrix (a
    ragged bottom row, a ragged right column, the corner) in one launch, several items per
    workgroup -- the write-out inside the last K-step with its stores under lane masks --
    for the int32 output and both 16-bit ones, with and without the one-item-per-workgroup
    launch, against the oracle; and the memory around C and D stays as it was."""
    m, n, k = shape
    a, b = make_operands(m, n, k, SEED_BASE + 7600 + m)
    ap, bp = pack_cpu(a), pack_cpu(b)
    rs, cs = make_scales(m, n, SEED_BASE + 7700 + m)
    c = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d, rs_d, cs_d = ap.to(DEV), bp.to(DEV), rs.to(DEV), cs.to(DEV)
    want16 = {out: oracle_mod.scale_round16(c, rs.numpy(), cs.numpy(), out) for _, out in DTYPES}
    pad = 4096    # elements either side of the output that must not change
    ran = 0
    for cfg, name in enumerate(qm.config_names()):
        if not name.startswith("q") or not qm.config_supports(cfg, m, n, k):
            continue
        bm, bn = (int(x) for x in name[1:].split("_")[0].split("x"))
        assert m % bm or n % bn, (name, shape)          # (some tile sticks out)
        for gm, spread in [(1, 0), (4, 0), (2, 1)]:
            code = cfg | (gm << 16) | (spread << 30)
            buf = torch.full((m * n + 2 * pad,), 0x7F7F7F7F, dtype=torch.int32, device=DEV)
            c_d = buf[pad:pad + m * n].view(m, n)
            qm.gemm_cfg(a_d, b_d, c_d, m, n, k, code)
            torch.cuda.synchronize()
            bad = oracle_mod.compare(c_d.cpu().numpy(), c)
            assert bad == -1, f"{name} group_m={gm} spread={spread}: first mismatch at flat index {bad} (row {bad // n}, column {bad % n})"
            assert (buf[:pad] == 0x7F7F7F7F).all() and (buf[pad + m * n:] == 0x7F7F7F7F).all(), name
            if not qm.config_has_scaled(cfg):
                continue
            for dtype, out in DTYPES:
                buf16 = torch.full((m * n + 2 * pad,), float("nan"), dtype=dtype, device=DEV)
                d_d = buf16[pad:pad + m * n].view(m, n)
                qm.gemm_scaled(a_d, b_d, d_d, m, n, k, rs_d, cs_d, code)
                torch.cuda.synchronize()
                assert (bits(d_d) == want16[out]).all(), f"{name} {dtype} group_m={gm} spread={spread}"
                assert torch.isnan(buf16[:pad]).all() and torch.isnan(buf16[pad + m * n:]).all(), name
        ran += 1
    assert ran >= 8
