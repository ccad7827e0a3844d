"""The paths of operands of 2 GiB and more, driven on small shapes: the library's limit above
which it cuts A into blocks of rows and B into blocks of its rows (blocks of columns of C,
written through a row stride) is lowered through qm_debug_set_operand_limit, so that every
kernel family writes through the stride -- int32 and scaled, strides that are no multiple
of four, strides of 2^21 and more, blocks of rows that are cut into blocks of columns in
turn -- against the CPU oracle.  The reference has no such path (shapes outside its table
are skipped, kernel.cu:340-385)."""
import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import SEED_BASE, make_operands, pack_cpu, poisoned_c

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture
def operand_limit():
    """Sets the limit for the test and restores 2 GiB - 1 afterwards, whatever happens."""
    def set_limit(nbytes):
        qm.debug_set_operand_limit(nbytes)
    yield set_limit
    qm.debug_set_operand_limit(0)


def _blocks(limit, k):
    return ((limit - 1) // (k // 2)) & ~255


def _check_both_outputs(oracle_mod, a, b, m, n, k, seed, expect_family=None):
    """quadmul_amd.gemm and gemm_scaled on (a, b) against the oracle; returns the int32 result."""
    ap, bp = pack_cpu(a), pack_cpu(b)
    want = oracle_mod.gemm_i4(ap.numpy(), bp.numpy())
    a_d, b_d = ap.to(DEV), bp.to(DEV)
    for ws in (True, None):
        c_d = poisoned_c(m, n, DEV)
        qm.gemm(a_d, b_d, c_d, m, n, k, workspace=ws)
        torch.cuda.synchronize()
        bad = oracle_mod.compare(c_d.cpu().numpy(), want)
        assert bad == -1, f"{m}x{n}x{k} workspace={ws}: first mismatch at flat index {bad} (row {bad // n}, column {bad % n})"
    g = torch.Generator().manual_seed(seed)
    rs, cs = torch.rand(m, generator=g) * 0.01 + 0.001, torch.rand(n, generator=g) + 0.5
    for dt, kind in ((torch.float16, oracle_mod.OUT_F16), (torch.bfloat16, oracle_mod.OUT_BF16)):
        d_d = torch.full((m, n), float("nan"), dtype=dt, device=DEV)
        qm.gemm_scaled(a_d, b_d, d_d, m, n, k, rs.to(DEV), cs.to(DEV))
        torch.cuda.synchronize()
        want16 = oracle_mod.scale_round16(want, rs.numpy(), cs.numpy(), kind)
        assert np.array_equal(d_d.view(torch.int16).cpu().numpy().view(np.uint16), want16), (m, n, k, dt)
    return want


# (m, the kernel family its blocks of columns run on)
FAMILIES = [(1, "v"), (2, "v"), (8, "d"), (16, "d"), (20, "p"), (40, "d"), (64, "d"), (100, "d"), (300, "d"), (1500, "q")]


@pytest.mark.parametrize("m,family", FAMILIES, ids=[f"m{m}" for m, _ in FAMILIES])
@pytest.mark.parametrize("n", [2100, 2051], ids=["ldc_mult_of_4", "ldc_odd"])
def test_blocks_of_columns_on_every_kernel_family(oracle_mod, operand_limit, m, family, n):
    """B above the limit, A below: blocks of 768 and 256 columns of C (the last one ragged)
    through a row stride of n -- a multiple of four (16-byte stores stay aligned where C is)
    or odd (element by element)."""
    k = 1024 if m <= 16 or m >= 1000 else 512
    limit = 800 * (k // 2) if m > 256 else 300 * (k // 2)
    if m * (k // 2) >= limit:   # (A must stay below: raise the limit just above it)
        limit = (m + 1) * (k // 2)
    operand_limit(limit)
    cols = _blocks(limit, k)
    assert 256 <= cols < n, (cols, n)
    # the blocks run on the family the test is about (what the library picks for one block)
    name = qm.config_name(qm.select_config(m, cols, k) & 0xFFFF)
    assert name[0] == family, (m, cols, k, name)
    a, b = make_operands(m, n, k, SEED_BASE + 9000 + 7 * m + n)
    assert qm.workspace_bytes(m, n, k) == 0          # blocks of columns: one launch each, no workspace
    _check_both_outputs(oracle_mod, a, b, m, n, k, SEED_BASE + 9100 + m)


def test_blocks_of_columns_on_the_generic_kernel(oracle_mod, operand_limit):
    """The generic kernel is not cut into blocks (it has 64-bit offsets and no operand limit):
    K % 32 != 0 keeps the whole call on it whatever the limit says."""
    m, n, k = 40, 1500, 70
    operand_limit(256 * (k // 2))
    assert qm.config_name(qm.select_config(m, n, k) & 0xFFFF) == "generic"
    a, b = make_operands(m, n, k, SEED_BASE + 9200)
    _check_both_outputs(oracle_mod, a, b, m, n, k, SEED_BASE + 9201)


@pytest.mark.parametrize("m", [2, 12, 48, 300], ids=lambda m: f"m{m}")
def test_row_stride_of_two_to_the_21_and_more(oracle_mod, operand_limit, m):
    """A row stride of C of 2^21 elements and more (the tile kernel's plain write-out addresses
    a tile through 32-bit byte offsets below that; beyond, its guarded path runs), on every
    family: a B of 2^21 + 37 rows of 32 bytes (64 for the tile kernel, which takes K from 128 on), cut
    into blocks of 2^19 columns."""
    k = 128 if m >= 256 else 64
    n = (1 << 21) + 37
    operand_limit((1 << 19) * (k // 2) + 1)
    assert _blocks((1 << 19) * (k // 2) + 1, k) == 1 << 19
    g = torch.Generator(device=DEV).manual_seed(SEED_BASE + 9300 + m)
    a_d = torch.randint(-128, 128, (m, k // 2), dtype=torch.int8, device=DEV, generator=g)
    b_d = torch.randint(-128, 128, (n, k // 2), dtype=torch.int8, device=DEV, generator=g)
    c_d = poisoned_c(m, n, DEV)
    qm.gemm(a_d, b_d, c_d, m, n, k)
    rs = torch.rand(m, device=DEV, generator=g) * 0.01 + 0.001
    cs = torch.rand(n, device=DEV, generator=g) + 0.5
    d_d = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
    qm.gemm_scaled(a_d, b_d, d_d, m, n, k, rs, cs)
    torch.cuda.synchronize()
    qm.debug_set_operand_limit(0)
    # every element against the library's own result without blocks (one launch, stride = n:
    # the path the other tests pin against the oracle) ...
    whole = poisoned_c(m, n, DEV)
    qm.gemm(a_d, b_d, whole, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(c_d, whole)
    # ... and the columns either side of every block boundary and the last ones against the oracle
    a_h = a_d.cpu().numpy()
    for c0 in [0] + [j * (1 << 19) - 20 for j in (1, 2, 3, 4)] + [n - 40]:
        ref = oracle_mod.gemm_i4(a_h, b_d[c0:c0 + 40].cpu().numpy())
        assert oracle_mod.compare(np.ascontiguousarray(c_d[:, c0:c0 + 40].cpu().numpy()), ref) == -1, (m, c0)
        ref16 = oracle_mod.scale_round16(ref, rs.cpu().numpy(), cs[c0:c0 + 40].cpu().numpy(), oracle_mod.OUT_F16)
        assert np.array_equal(np.ascontiguousarray(d_d[:, c0:c0 + 40].view(torch.int16).cpu().numpy()).view(np.uint16), ref16), (m, c0)


@pytest.mark.parametrize("shape", [(1300, 1400, 256), (600, 2000, 512 + 32), (2600, 530, 128)], ids=lambda s: "x".join(map(str, s)))
def test_blocks_of_rows_cut_into_blocks_of_columns(oracle_mod, operand_limit, shape):
    """A and B both above the limit: blocks of rows of A, each cut into blocks of columns in
    turn; the workspace the call asks for is that of its largest block."""
    m, n, k = shape
    limit = 520 * (k // 2)
    operand_limit(limit)
    blk = _blocks(limit, k)
    assert blk == 512 and m > blk and n > blk
    a, b = make_operands(m, n, k, SEED_BASE + 9400 + m)
    assert qm.workspace_bytes(m, n, k) == 0
    _check_both_outputs(oracle_mod, a, b, m, n, k, SEED_BASE + 9401 + m)


def test_blocks_of_rows_keep_their_workspace_use(oracle_mod, operand_limit):
    """A above the limit, B below it: each block of rows is a call of its own and may split K
    through the workspace; the call asks for what its largest block uses."""
    m, n, k = 2600, 1024, 28672
    limit = 1300 * (k // 2)
    operand_limit(limit)
    assert _blocks(limit, k) == 1280
    need = qm.workspace_bytes(m, n, k)
    assert need == max(qm.workspace_bytes(1280, n, k), qm.workspace_bytes(m % 1280, n, k)) > 0
    assert (qm.select_config(1280, n, k) >> 24) & 0x3F > 1
    a, b = make_operands(m, n, k, SEED_BASE + 9500)
    _check_both_outputs(oracle_mod, a, b, m, n, k, SEED_BASE + 9501)


def test_the_limit_is_restored():
    assert qm.debug_set_operand_limit(0) == 2 ** 31 - 1
