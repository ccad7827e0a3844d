"""qm_gemm_i4_static, the entry point that allocates nothing: its scratch memory (partial
tiles of a K split, zero-padded operand copies) is an array inside the library.  Called
through the C ABI and compared bit for bit with qm_gemm_i4_ws on a caller's workspace, the
existing entry point whose kernels it shares -- on calls in a row that reuse the array, the
later ones with smaller inputs -- and with the CPU oracle where that takes seconds."""
import ctypes

import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import SEED_BASE, make_operands, pack_cpu, poisoned_c

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _static(a_d, b_d, m, n, k):
    """One call through the C ABI, on the current stream; the status is returned as it is."""
    c_d = poisoned_c(m, n, DEV)
    st = qm.library().qm_gemm_i4_static(a_d.data_ptr(), b_d.data_ptr(), c_d.data_ptr(), m, n, k,
                                        torch.cuda.current_stream().cuda_stream)
    return st, c_d


def _with_workspace(a_d, b_d, m, n, k):
    need = qm.workspace_bytes(m, n, k)
    ws = torch.full((max(need, 16),), 0x5A, dtype=torch.uint8, device=DEV)
    c_d = poisoned_c(m, n, DEV)
    st = qm.library().qm_gemm_i4_ws(a_d.data_ptr(), b_d.data_ptr(), c_d.data_ptr(), m, n, k,
                                    torch.cuda.current_stream().cuda_stream, qm.CFG_AUTO, ws.data_ptr() if need else None, need)
    assert st == 0
    return c_d, need


# (shape, what the scratch array holds for it), largest use first: every later call finds the
# array full of an earlier call's data
CALLS = [
    ((256, 8192, 28672), "partial tiles of a K split, 32 MiB"),
    ((640, 4096, 20480), "partial tiles of a K split of three, 30 MiB"),
    ((2048, 4096, 4100), "zero-padded copies of A and B"),
    ((384, 3072, 20480), "partial tiles of a K split of three, 13 MiB"),
    ((200, 300, 1152), "nothing (one launch, no scratch)"),
]


def test_static_scratch_matches_caller_workspace_on_calls_in_a_row(oracle_mod):
    print("qm_gemm_i4_static vs qm_gemm_i4_ws:", flush=True)
    free_before = None
    for i, ((m, n, k), what) in enumerate(CALLS):
        print(f"  call {i}: {m}x{n}x{k} ({what})", flush=True)
        a, b = make_operands(m, n, k, SEED_BASE + 7000 + i)
        ap, bp = pack_cpu(a), pack_cpu(b)
        a_d, b_d = ap.to(DEV), bp.to(DEV)
        want, need = _with_workspace(a_d, b_d, m, n, k)
        assert (need > 0) == (not what.startswith("nothing")), (m, n, k, need)
        assert need <= qm.STATIC_SCRATCH_BYTES
        torch.cuda.synchronize()
        if i >= 1:
            free_before = torch.cuda.mem_get_info()[0]
        st, got = _static(a_d, b_d, m, n, k)
        assert st == 0, qm.library().qm_status_string(st)
        torch.cuda.synchronize()
        if i >= 1:
            # the device's free memory is what it was before the call (the first call may load
            # the library's device code, which holds the array)
            assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(got, want), f"{m}x{n}x{k}: differs from qm_gemm_i4_ws"
        # and both against an independent product: exact fp32 (integers below 2^24) for every
        # element, the oracle for a sample of rows (all rows of the small shape)
        exact = (a.to(DEV).float() @ b.to(DEV).float().t()).to(torch.int32)
        assert torch.equal(got, exact), f"{m}x{n}x{k}: differs from the exact fp32 product"
        rows = np.arange(m, dtype=np.int32) if m * n * k <= 2 ** 27 else np.linspace(0, m - 1, 4).astype(np.int32)
        assert (got.cpu().numpy()[rows] == oracle_mod.gemm_i4_rows(ap.numpy(), bp.numpy(), rows)).all()


def test_static_scratch_twice_on_one_stream_then_smaller(oracle_mod):
    # the same array back to back without a synchronisation in between: stream order is all
    # that separates the second call's writes from the first call's reads
    (m1, n1, k1), (m2, n2, k2) = (256, 8192, 28672), (640, 4096, 20480)
    a1, b1 = make_operands(m1, n1, k1, SEED_BASE + 7100)
    a2, b2 = make_operands(m2, n2, k2, SEED_BASE + 7101)
    d1 = (pack_cpu(a1).to(DEV), pack_cpu(b1).to(DEV))
    d2 = (pack_cpu(a2).to(DEV), pack_cpu(b2).to(DEV))
    torch.cuda.synchronize()
    print(f"  back to back: {m1}x{n1}x{k1} then {m2}x{n2}x{k2}", flush=True)
    st1, c1 = _static(*d1, m1, n1, k1)
    st2, c2 = _static(*d2, m2, n2, k2)
    st3, c3 = _static(*d1, m1, n1, k1)
    assert (st1, st2, st3) == (0, 0, 0)
    torch.cuda.synchronize()
    w1, _ = _with_workspace(*d1, m1, n1, k1)
    w2, _ = _with_workspace(*d2, m2, n2, k2)
    torch.cuda.synchronize()
    assert torch.equal(c1, w1) and torch.equal(c2, w2) and torch.equal(c3, w1)
    rows = np.array([0, 77, 127], dtype=np.int32)
    assert (c2.cpu().numpy()[rows] == oracle_mod.gemm_i4_rows(d2[0].cpu().numpy(), d2[1].cpu().numpy(), rows)).all()


def test_static_scratch_rejects_what_does_not_fit():
    # zero-padded copies of 2 x 16384 x 4096 bytes: 128 MiB; nothing is enqueued, the operands are never touched
    m = n = 16384
    k = 8100
    assert qm.workspace_bytes(m, n, k) > qm.STATIC_SCRATCH_BYTES
    one = ctypes.c_void_p(4096)
    assert qm.library().qm_gemm_i4_static(one, one, one, m, n, k, None) == -7
    assert b"scratch" in qm.library().qm_status_string(-7)
    with pytest.raises(qm.QuadmulError, match="scratch"):
        qm._check(-7, "qm_gemm_i4_static")
