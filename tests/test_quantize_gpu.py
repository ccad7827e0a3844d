"""GPU parity of the fused quantise + pack kernel (through the C ABI) against the CPU oracle:
packed bytes and scales bit-exact; then the whole int4 linear layer end to end."""
import numpy as np
import pytest
import torch

import quadmul_amd as qm
from util import SEED_BASE

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
SHAPES = [(1, 2), (3, 6), (7, 30), (16, 64), (33, 130), (64, 4096), (5, 4104), (9, 8192), (4, 16384), (3, 16392), (2, 40960), (257, 1184), (0, 64), (5, 0)]


def make_x(rows, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((rows, k), generator=g) * (torch.rand((rows, 1), generator=g) * 20 + 0.01)
    if rows > 2:
        x[1] = 0                      # an all-zero row
        x[2] = torch.round(x[2])      # exact ties after scaling are likely here
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_quantize_pack_matches_oracle(oracle_mod, shape, dtype):
    rows, k = shape
    x = make_x(rows, k, dtype, SEED_BASE + 8000 + rows + k)
    want_p, want_s = oracle_mod.quantize_pack(x.to(torch.float32).numpy())
    packed, scales = qm.quantize_pack(x.to(DEV))
    torch.cuda.synchronize()
    assert packed.shape == (rows, k // 2) and packed.dtype == torch.int8 and scales.shape == (rows,)
    assert (scales.cpu().numpy() == want_s).all()
    got = packed.cpu().numpy().view(np.uint8)
    bad = np.flatnonzero(got != want_p)
    assert bad.size == 0, f"{bad.size} packed bytes differ, first at {bad[0]}: got {got.flat[bad[0]]:#04x} want {want_p.flat[bad[0]]:#04x}"


def test_quantize_pack_unaligned_input(oracle_mod):
    rows, k = 6, 72
    x = make_x(rows, k, torch.float16, SEED_BASE + 8100)
    buf = torch.zeros(rows * k + 8, dtype=torch.float16, device=DEV)
    view = buf[1:1 + rows * k].view(rows, k)      # 2-byte aligned only: the element-wise kernel
    view.copy_(x)
    want_p, want_s = oracle_mod.quantize_pack(x.to(torch.float32).numpy())
    packed, scales = qm.quantize_pack(view)
    torch.cuda.synchronize()
    assert (packed.cpu().numpy().view(np.uint8) == want_p).all() and (scales.cpu().numpy() == want_s).all()


def test_int4_linear_layer_end_to_end(oracle_mod):
    """activations -> quantize_pack -> gemm_scaled(row_scale = activation scales, col_scale =
    weight scales) against the oracle's chain of the same three steps (bit-exact), and against
    the float product (within the quantisation error)."""
    m, n, k = 96, 320, 1024
    g = torch.Generator().manual_seed(SEED_BASE + 8200)
    x = (torch.randn((m, k), generator=g) * 0.5).to(torch.float16)
    w = (torch.randn((n, k), generator=g) * 0.05).to(torch.float16)
    import quadmul

    xq, xs = quadmul.quantize_pack(x.to(DEV))   # the extension module's entry point
    wq, ws = qm.quantize_pack(w.to(DEV))        # the ctypes binding of the same C function
    y = torch.empty((m, n), dtype=torch.float16, device=DEV)
    qm.gemm_scaled(xq, wq, y, m, n, k, xs, ws)
    torch.cuda.synchronize()
    oxq, oxs = oracle_mod.quantize_pack(x.float().numpy())
    owq, ows = oracle_mod.quantize_pack(w.float().numpy())
    want = oracle_mod.scale_round16(oracle_mod.gemm_i4(oxq, owq), oxs, ows, oracle_mod.OUT_F16)
    assert (y.view(torch.int16).cpu().numpy().view(np.uint16) == want).all()
    ref = x.float() @ w.float().t()
    err = (y.float().cpu() - ref).norm() / ref.norm()
    assert err < 0.25, err  # int4 x int4 with per-row scales: about 15 % relative error on gaussian data


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_w4a4_linear_module(oracle_mod, out_dtype):
    """The module form of the same chain: leading dimensions flattened, weights quantised once,
    bias added to the rounded output; bit-exact against the oracle's chain; no rows -> no launch."""
    from quadmul_amd.linear import W4A4Linear

    n, k = 272, 1056
    g = torch.Generator().manual_seed(SEED_BASE + 8300)
    x = (torch.randn((3, 5, k), generator=g) * 0.7).to(torch.bfloat16)
    w = (torch.randn((n, k), generator=g) * 0.03).to(torch.float32)
    bias = torch.randn((n,), generator=g).to(out_dtype)
    layer = W4A4Linear.from_float(w.to(DEV), bias.to(DEV), out_dtype)
    assert (layer.in_features, layer.out_features) == (k, n) and "bias=True" in repr(layer)
    y = layer(x.to(DEV))
    torch.cuda.synchronize()
    assert y.shape == (3, 5, n) and y.dtype == out_dtype
    oxq, oxs = oracle_mod.quantize_pack(x.reshape(-1, k).float().numpy())
    owq, ows = oracle_mod.quantize_pack(w.numpy())
    out = oracle_mod.OUT_F16 if out_dtype == torch.float16 else oracle_mod.OUT_BF16
    d = oracle_mod.scale_round16(oracle_mod.gemm_i4(oxq, owq), oxs, ows, out)
    want = torch.from_numpy(d.view(np.int16)).view(out_dtype) + bias   # one rounded add in the output type
    assert torch.equal(y.reshape(-1, n).cpu().view(torch.int16), want.view(torch.int16))
    # the state dict round-trips through the constructor's arguments
    again = W4A4Linear(layer.weight_packed, layer.weight_scale, layer.bias, out_dtype)
    assert torch.equal(again(x.to(DEV)), y)
    assert layer(torch.empty((0, k), dtype=torch.float16, device=DEV)).shape == (0, n)
    with pytest.raises(qm.QuadmulError):
        layer(torch.zeros((2, k + 2), dtype=torch.float16, device=DEV))


def test_linear_chain_through_dispatcher_ops_traced(oracle_mod):
    """quantize_pack and gemm_scaled as dispatcher ops: the whole linear chain stays in one
    traced graph (aot_eager: fake tensors go through the Meta implementations) and gives the
    oracle's bits."""
    import quadmul  # noqa: F401

    m, n, k = 48, 96, 512
    g = torch.Generator().manual_seed(SEED_BASE + 8400)
    x = (torch.randn((m, k), generator=g) * 0.5).to(torch.float16)
    w = (torch.randn((n, k), generator=g) * 0.05).to(torch.float16)
    wq, ws = torch.ops.quadmul.quantize_pack(w.to(DEV))

    def fn(x_, wq_, ws_):
        xq, xs = torch.ops.quadmul.quantize_pack(x_)
        y = torch.empty((m, n), dtype=torch.float16, device=x_.device)
        torch.ops.quadmul.gemm_scaled(xq, wq_, y, m, n, k, xs, ws_)
        return y

    y = torch.compile(fn, backend="aot_eager", fullgraph=True)(x.to(DEV), wq, ws)
    torch.cuda.synchronize()
    oxq, oxs = oracle_mod.quantize_pack(x.float().numpy())
    owq, ows = oracle_mod.quantize_pack(w.float().numpy())
    want = oracle_mod.scale_round16(oracle_mod.gemm_i4(oxq, owq), oxs, ows, oracle_mod.OUT_F16)
    assert (y.view(torch.int16).cpu().numpy().view(np.uint16) == want).all()
