"""No-GPU checks of the C-ABI library and the host-side interface: the library
loads, exports every symbol include/qm_abi.h declares, rejects bad arguments with
the documented status codes, and selects sensible configurations.  No kernel is
launched here."""
import ctypes
import os
import re

import pytest
import torch

import quadmul_amd as qm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "qm_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = qm.library()
    syms = declared_symbols()
    assert set(syms) == set(qm.ABI_SYMBOLS)
    for s in syms:
        assert hasattr(lib, s), s


def test_extension_module_imports_and_mirrors_reference_entry_point():
    import quadmul  # the drop-in module name (setup.py:8,11 of the reference)

    assert callable(quadmul.gemm)
    assert "Int4xInt4 Matrix Multiplication Kernel" in quadmul.gemm.__doc__  # extension.cpp:28
    assert quadmul.num_configs() == qm.num_configs()
    assert callable(quadmul.gemm_scaled)


def test_dispatcher_op_is_registered_with_a_mutation_schema():
    import torch
    import quadmul  # noqa: F401  (registers torch.ops.quadmul.gemm)

    schema = torch.ops.quadmul.gemm.default._schema
    assert [a.name for a in schema.arguments] == ["a", "b", "c", "m", "n", "k"]
    assert schema.arguments[2].alias_info is not None and schema.arguments[2].alias_info.is_write
    assert len(schema.returns) == 0
    scaled = torch.ops.quadmul.gemm_scaled.default._schema
    assert [a.name for a in scaled.arguments] == ["a", "b", "d", "m", "n", "k", "row_scale", "col_scale"]
    assert scaled.arguments[2].alias_info is not None and scaled.arguments[2].alias_info.is_write
    # the Meta kernel lets a tracer run the op without data
    a = torch.empty((4, 16), dtype=torch.int8, device="meta")
    c = torch.empty((4, 4), dtype=torch.int32, device="meta")
    assert torch.ops.quadmul.gemm(a, a, c, 4, 4, 32) is None
    # no CPU kernel: the product path is the GPU one only
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.quadmul.gemm(torch.zeros((4, 16), dtype=torch.int8), torch.zeros((4, 16), dtype=torch.int8),
                               torch.zeros((4, 4), dtype=torch.int32), 4, 4, 32)


def test_status_codes_without_a_gpu():
    lib = qm.library()
    one = ctypes.c_void_p(4096)  # never dereferenced: the checks come first
    assert lib.qm_gemm_i4(one, one, one, 4, 4, 3, None) == -2      # odd k
    assert lib.qm_gemm_i4(one, one, one, -1, 4, 4, None) == -2     # negative m
    assert lib.qm_gemm_i4(None, one, one, 4, 4, 4, None) == -1     # null A
    assert lib.qm_gemm_i4(one, one, None, 4, 4, 4, None) == -1     # null C
    assert lib.qm_gemm_i4(one, one, ctypes.c_void_p(4098), 4, 4, 4, None) == -5
    assert lib.qm_gemm_i4(None, None, None, 0, 4, 4, None) == 0    # empty: nothing to do
    assert lib.qm_gemm_i4(None, None, None, 4, 0, 4, None) == 0
    assert lib.qm_gemm_i4_cfg(one, one, one, 4, 4, 4, None, 9999) == -3
    assert lib.qm_gemm_i4_cfg(one, one, one, 128, 128, 30, None, qm.config_id("q128x128_w2x2_s7o1")) == -3   # K % 32 != 0
    assert lib.qm_gemm_i4_cfg(one, one, one, 256, 256, 96, None, qm.config_id("q256x256_w2x2_s4o1")) == -3   # a single short K-step
    # the entry point on the library's own scratch array: same checks, and a call that would
    # need more than the array holds is refused before anything touches the GPU
    assert lib.qm_gemm_i4_static(one, one, one, 4, 4, 3, None) == -2
    assert lib.qm_gemm_i4_static(one, one, None, 4, 4, 4, None) == -1
    assert lib.qm_gemm_i4_static(None, None, None, 0, 4, 4, None) == 0
    assert qm.workspace_bytes(16384, 16384, 8100) > qm.STATIC_SCRATCH_BYTES
    assert lib.qm_gemm_i4_static(one, one, one, 16384, 16384, 8100, None) == -7
    assert lib.qm_pack_i4(one, one, 4, 3, None) == -2
    assert lib.qm_pack_i4(None, None, 0, 8, None) == 0
    assert lib.qm_unpack_i4(None, one, 4, 8, None) == -1
    # the scaled GEMM and the quantiser reject bad arguments before they touch the GPU too
    assert lib.qm_gemm_i4_scaled(one, one, one, 4, 4, 4, None, None, 7, None) == -6        # unknown output type
    assert lib.qm_gemm_i4_scaled(one, one, one, 4, 4, 3, None, None, 1, None) == -2
    assert lib.qm_gemm_i4_scaled(one, one, None, 4, 4, 4, None, None, 1, None) == -1
    assert lib.qm_gemm_i4_scaled(one, one, ctypes.c_void_p(4097), 4, 4, 4, None, None, 2, None) == -5
    assert lib.qm_gemm_i4_scaled(None, None, None, 0, 4, 4, None, None, 1, None) == 0
    assert lib.qm_gemm_i4_scaled_cfg(one, one, one, 64, 64, 128, None, None, 1, None, qm.config_id("q256x128_w2x2_s3o2")) == -3   # no scaled output
    assert lib.qm_gemm_i4_scaled_cfg(one, one, one, 256, 256, 256, None, None, 1, None, qm.config_id("q256x256_w2x2_s4o1") | (2 << 24)) == -3
    assert lib.qm_quantize_pack_i4(one, 9, one, one, 4, 8, None) == -6
    assert lib.qm_quantize_pack_i4(one, 1, one, one, 4, 7, None) == -2
    assert lib.qm_quantize_pack_i4(one, 1, one, None, 4, 8, None) == -1
    assert lib.qm_quantize_pack_i4(ctypes.c_void_p(4097), 1, one, one, 4, 8, None) == -5
    assert lib.qm_quantize_pack_i4(None, 3, None, None, 0, 8, None) == 0
    # the forms with a workspace: same checks; the workspace itself is optional
    assert lib.qm_gemm_i4_ws(one, one, one, 4, 4, 3, None, -1, None, 0) == -2
    assert lib.qm_gemm_i4_ws(one, one, None, 4, 4, 4, None, -1, one, 1 << 20) == -1
    assert lib.qm_gemm_i4_ws(None, None, None, 0, 4, 4, None, -1, None, 0) == 0
    assert lib.qm_gemm_i4_ws(one, one, one, 64, 64, 512, None, qm.config_id("s4x1_w8_u2") | (2 << 24), one, 1 << 20) == -3   # only the pipelined kernel splits K
    assert lib.qm_gemm_i4_scaled_ws(one, one, one, 4, 4, 4, None, None, 7, None, -1, None, 0) == -6
    assert lib.qm_gemm_i4_scaled_ws(one, one, one, 256, 256, 512, None, None, 1, None, qm.config_id("q256x256_w2x2_s4o1") | (2 << 24), one, 4096) == -3
    has = [qm.config_has_scaled(i) for i in range(qm.num_configs())]
    assert has[qm.config_id("generic")] and has[qm.config_id("q256x256_w2x2_s4o1")] and has[qm.config_id("s1x1_w8_u4")]
    assert not has[qm.config_id("q256x128_w2x2_s3o2")]
    for code in (0, -1, -2, -3, -4, -5, -6):
        assert lib.qm_status_string(code)
    assert b"gfx950" in lib.qm_version()


def test_workspace_sizes():
    q128 = qm.config_id("q128x128_w2x2_s7o1")
    # one padded int32 tile per (split, tile): 2 x 3 tiles of 128 x 128, 4 splits
    assert qm.workspace_bytes(200, 300, 4096, q128 | (4 << 24)) == 4 * 6 * 128 * 128 * 4
    # splits without work do not count: 3 K-steps cannot feed 8 splits
    assert qm.workspace_bytes(200, 300, 384, q128 | (8 << 24)) == 3 * 6 * 128 * 128 * 4
    assert qm.workspace_bytes(200, 300, 4096, q128) == 0                       # no split asked for
    assert qm.workspace_bytes(16, 300, 4096, qm.config_id("s1x1_w8_u4") | (4 << 24)) == 0
    assert qm.workspace_bytes(8192, 8192, 8192) == 0                           # plenty of tiles
    code = qm.select_config(256, 8192, 28672)
    assert (code >> 24) & 0x3F > 1
    assert qm.workspace_bytes(256, 8192, 28672) == qm.workspace_bytes(256, 8192, 28672, code) > 0
    assert qm.workspace_bytes(256, 8192, 28672, scaled=True) > 0
    assert qm.workspace_bytes(128, 8192, 28672) == 0                          # one round of 64 x 64 blocks of the wave-level kernel
    assert qm.workspace_bytes(0, 8192, 28672) == 0 and qm.workspace_bytes(128, 8192, 3) == 0
    # large shapes with K % 32 != 0 (or unaligned operands): room for copies of A and B with rows
    # padded to whole K-steps
    assert qm.workspace_bytes(4096, 4096, 4162) == 2 * 4096 * (4224 // 2)
    assert qm.workspace_bytes(4096, 4096, 4160, ptr_align=2) == 2 * 4096 * (4224 // 2)
    assert qm.workspace_bytes(4096, 4096, 4160) == 0         # K % 32 == 0: the pipelined kernel takes it as it is
    assert qm.workspace_bytes(60, 70, 4162) == 0             # too small to pay for the copies
    assert qm.workspace_bytes(4096, 4096, 4162, qm.config_id("generic")) == 0   # explicit configuration: as asked


def test_version_names_the_compiler():
    v = qm.version()
    assert v.startswith("quadmul-amd") and "gfx950" in v and "HIP version" in v, v


def test_config_registry():
    names = qm.config_names()
    assert names[0] == "generic" and len(names) == len(set(names))
    assert any(n.startswith("q64x64") for n in names) and any(n.startswith("s1x1") for n in names)
    assert any(n.startswith("q256x256") for n in names) and any(n.startswith("v1x1") for n in names)
    for i, n in enumerate(names):
        assert qm.config_id(n) == i
    with pytest.raises(qm.QuadmulError):
        qm.config_name(len(names))


def test_selection_rules():
    name = lambda m, n, k, al=256: qm.config_name(qm.select_config(m, n, k, al) & 0xFFFF)
    assert name(8192, 8192, 8192).startswith("q")   # pipelined 16x16x64 kernel: K % 128 == 0
    assert name(4096, 4096, 4096).startswith("q")
    assert name(4096, 4096, 4096 + 32).startswith("q")  # K % 32 == 0: the pipelined kernel with a short last K-step
    # a single short K-step: nothing for the pipelined kernel to overlap it with; 32 x 32 blocks of the wave-level kernel
    assert name(4096, 4096, 96) == "d2x2_w1_r1" and name(300, 300, 64) == "d2x2_w8_r1" and name(4096, 4096, 128).startswith("q")
    assert qm.workspace_bytes(4096, 4096, 96) == 0
    # up to 64 rows: the wave-level split-K kernels; 3..16 rows stream their operands global ->
    # LDS, with a persistent grid and A resident in registers ("p") while the waves hold all of
    # K, the plain form ("d") beyond; from 33 rows the "d" form's grid walks over blocks of 32 rows
    assert name(16, 4096, 4096) == "p1x1_w8_r2k2" and name(64, 4096, 4096) == "d2x2_w8_r1"
    assert name(1, 4096, 4096) == "v1x1_w4_u8" and name(1, 11008, 2048) == "v1x1_w8_u4" and name(2, 5120, 5120) == "v2x1_w16_u2"   # dot-product kernel
    assert name(1, 4096, 8192) == "v1x1_w16_u2" and name(2, 4096, 4096) == "v2x1_w8_u4"
    # one or two rows on a K of 8192 and many columns: the persistent MFMA kernel is ahead of the dot kernel;
    # four waves of eight chunk pairs again on a very long K
    assert name(1, 8192, 8192) == "p1x1_w16_r2k2" and name(2, 57344, 8192) == "p1x1_w16_r2k2" and name(1, 8192, 28672) == "v1x1_w4_u8"
    # a very long K on up to 16 rows: 32 columns per workgroup; tens of thousands of columns on up to 32 rows: one wave per workgroup
    assert name(16, 8192, 28672) == "d1x2_w8_r2" and name(32, 57344, 8192) == "d2x2_w1_r1"
    assert name(9, 28672, 14336) == "d1x1_w16_r1" and name(9, 11008, 8192) == "p1x1_w16_r2k2" and name(12, 2048, 2048) == "d1x1_w16_r1"
    assert name(3, 28672, 2048) == "p1x1_w8_r2k2" and name(16, 4096, 8192) == "d1x1_w16_r1"
    assert name(32, 11008, 4096) == "p2x1_w8_r2k2" and name(24, 4096, 2048) == "p2x1_w16_r2k1"
    assert name(24, 4096, 8192) == "d2x1_w16_r1" and name(32, 28672, 8192) == "d2x2_w8_r1" and name(20, 2048, 8192) == "d1x1_w16_r1"
    assert name(40, 4096, 14336) == "d2x2_w8_r1" and name(64, 2048, 4096) == "d2x1_w16_r1"
    # 33 rows and more on enough columns: 64 x 32 and 64 x 64 blocks in one round of workgroups
    assert name(64, 8192, 4096) == "d4x2_w8_r1" and name(64, 11008, 4096) == "d4x4_w8_r1" and name(40, 16384, 8192) == "d4x4_w8_r1"
    # From 65 rows (and 33 to 64 on a short K or very many columns) the fitted cost model
    # chooses, among the tiles of the pipelined kernel and the blocks of the wave-level one.
    # A few hundred rows on few columns: 32 x 32 blocks (96 rows are three of them, not two of 64)
    assert name(128, 2048, 8192) == "d2x2_w8_r1" and name(96, 2048, 4096) == "d2x2_w8_r1" and name(96, 11008, 4096) == "d2x2_w8_r1"
    assert name(72, 2560, 8192) == "d2x2_w8_r1" and name(96, 5120, 3072) == "d2x4_w8_r1"
    # ... 64 x 64, 32 x 64 or 64 x 32 blocks, one workgroup per CU, where that makes one round that fills most of the device
    assert name(128, 8192, 4096) == "d4x4_w8_r1" and name(256, 4096, 4096) == "d4x4_w8_r1" and name(512, 2048, 8192) == "d4x4_w8_r1"
    assert name(128, 4096, 8192) == "d2x4_w8_r1" and name(192, 4096, 4096) == "d4x4_w8_r1" and name(256, 2048, 4096) == "d2x4_w8_r1"
    # ... or up to two rounds and a half of 64 x 64 blocks on four waves, two workgroups to a CU; tiles beyond
    assert name(256, 8192, 4096) == "d4x4_w4_r1" and name(512, 4096, 4096) == "d4x4_w4_r1" and name(64, 40000, 4096) == "d4x4_w4_r1"
    assert name(128, 4096, 512) == "d4x2_w8_r1" and name(300, 300, 256) == "d1x1_w4_r4"
    assert name(512, 8192, 4096).startswith("q") and name(384, 8192, 28672).startswith("q") and name(1000, 4096, 4096).startswith("q")
    d22 = qm.config_id("d2x2_w8_r1")
    assert qm.config_supports(d22, 1000, 4096, 4096) and not qm.config_supports(qm.config_id("p2x1_w8_r2k2"), 33, 4096, 4096)
    # a persistent "p" configuration only takes the K its waves hold in registers
    pk = qm.config_id("p1x1_w8_r2k2")
    assert qm.config_supports(pk, 16, 4096, 4096) and not qm.config_supports(pk, 16, 4096, 4096 + 32) and not qm.config_supports(pk, 17, 4096, 4096)
    assert name(64, 28672, 14336) == "d4x4_w4_r1" and name(64, 40000, 14336) == "d4x4_w4_r1"
    # few tiles, long K: the pipelined kernel with K split over several workgroups per tile
    code = qm.select_config(256, 8192, 28672)
    assert qm.config_name(code & 0xFFFF).startswith("q") and (code >> 24) & 0x3F > 1
    assert (qm.select_config(8192, 8192, 8192) >> 24) & 0x3F == 1
    # ... which the table's rows were measured with: without a workspace (the plain 7-argument
    # call) such a row's second, unsplit choice runs (measured without one); the cost model
    # for untabled shapes prices the atomics of a split without a workspace and keeps none here
    for (m, n, k) in [(256, 8192, 28672), (512, 8192, 28672), (384, 8192, 28672), (640, 4096, 20480), (384, 3072, 20480)]:
        with_ws, without = qm.select_config_ex(m, n, k, workspace=True), qm.select_config_ex(m, n, k, workspace=False)
        assert (with_ws >> 24) & 0x3F > 1 and with_ws == qm.select_config(m, n, k)
        assert qm.config_name(without & 0xFFFF).startswith(("q", "d2x2", "d4x4")) and (without >> 24) & 0x3F == 1, (m, n, k)
    assert qm.config_name(qm.select_config_ex(512, 8192, 28672, workspace=False) & 0xFFFF) == "q128x128_w2x2_s9o1"
    # scaled output, no workspace, long K with a short last K-step: a configuration that has
    # the output form, never the generic kernel
    for (m, n, k) in [(256, 256, 28704), (128, 8192, 28672 + 32), (512, 4096, 14336 + 96), (640, 4096, 14336 + 32)]:
        code = qm.select_config_ex(m, n, k, workspace=False, scaled=True)
        assert qm.config_name(code & 0xFFFF)[0] in "qd" and (code >> 24) & 0x3F == 1, (m, n, k)
        assert qm.config_has_scaled(code & 0xFFFF)
    assert name(100, 100, 30) == "generic"          # K % 32 != 0: no 16-byte chunks
    assert name(128, 128, 4096, 4) == "generic"     # operands not 16-byte aligned
    assert name(128, 128, 262144) == "generic"      # beyond the exact range of the x16 widening
    gid, sk = qm.config_id("generic"), qm.config_id("s1x1_w8_u4")
    assert qm.config_supports(gid, 3, 5, 2, 1)
    assert qm.config_supports(sk, 16, 4096, 4096) and not qm.config_supports(sk, 17, 4096, 4096)
    assert not qm.config_supports(sk, 16, 4096, 4098)


def test_host_checks_reject_bad_tensors():
    a = torch.zeros(4, 4, dtype=torch.int8)
    c = torch.zeros(4, 4, dtype=torch.int32)
    with pytest.raises(qm.QuadmulError):
        qm.gemm(a, a, c, 4, 4, 8)  # CPU tensors
    import quadmul
    with pytest.raises(RuntimeError):
        quadmul.gemm(a, a, c, 4, 4, 8)


def test_cpu_pack_unpack_mirror_reference_semantics():
    from util import make_values, pack_cpu

    v = make_values(9, 64, 3)
    p = qm.pack_int4(v)
    assert p.dtype == torch.int8 and p.shape == (9, 32)
    assert torch.equal(p, pack_cpu(v))
    assert torch.equal(qm.unpack_int4(p), v)
    with pytest.raises(qm.QuadmulError):
        qm.pack_int4(torch.zeros(2, 3, dtype=torch.int8))


def test_w4a4_linear_argument_checks():
    """Constructor checks of the linear-layer caller (no GPU: nothing is launched)."""
    import torch
    from quadmul_amd.linear import W4A4Linear

    wq = torch.zeros((8, 16), dtype=torch.int8)
    ws = torch.ones(8, dtype=torch.float32)
    layer = W4A4Linear(wq, ws, torch.zeros(8), torch.bfloat16)
    assert (layer.in_features, layer.out_features) == (32, 8) and layer.bias.dtype == torch.bfloat16
    assert set(layer.state_dict()) == {"weight_packed", "weight_scale", "bias"}
    for bad in (lambda: W4A4Linear(wq.float(), ws), lambda: W4A4Linear(wq, ws[:4]), lambda: W4A4Linear(wq, ws.double()),
                lambda: W4A4Linear(wq, ws, torch.zeros(7)), lambda: W4A4Linear(wq, ws, None, torch.float32)):
        with pytest.raises(qm.QuadmulError):
            bad()


# --------------------------------------------------------------------------
# Committed measurements must describe the kernels the library chooses today: a table row
# retuned after the last profile / benchmark run fails here instead of leaving a stale figure.
# --------------------------------------------------------------------------
def _bench_module():
    import importlib.util

    spec = importlib.util.spec_from_file_location("qm_bench_for_tests", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_every_profile_summary_is_of_the_configuration_the_library_chooses():
    bench = _bench_module()
    profs = bench.profile_summaries()
    assert profs, "no rocprofv3 summaries under profiles/"
    for name, prof in profs.items():
        m, n, k = prof["shape"]
        scaled = name.endswith("_scaled_f16")
        chosen = qm.config_name(qm.select_config_ex(m, n, k, scaled=scaled) & 0xFFFF)
        assert prof["config"] == chosen, f"{prof['path']} profiled {prof['config']}, the library now chooses {chosen} for {m}x{n}x{k}"
        # the file is named for the kernel, the configuration and the workload it covers
        assert os.path.basename(prof["path"]).endswith(f"{prof['config']}__{name}.md"), prof["path"]
        total = prof["traffic"]
        assert 0.9 * bench.algorithmic_bytes(m, n, k) * (0.5 if scaled else 1.0) <= total <= 4 * bench.algorithmic_bytes(m, n, k), prof["path"]


def test_bench_reads_traffic_from_the_summaries_for_every_workload_of_the_contract():
    bench = _bench_module()
    for name, (_, m, n, k, bound) in bench.WORKLOADS.items():
        chosen = qm.config_name(qm.select_config(m, n, k) & 0xFFFF)
        traffic, source = bench.profiled_traffic(name, m, n, k, chosen)
        assert traffic is not None, f"{name}: {source}"
        assert source.endswith(".md)") and f"__{name}.md" in source
        if bound == "hbm":   # the HBM-fed figure these entries quote has a summary of its own
            traffic_rot, source_rot = bench.profiled_traffic(name + "_rotating_b", m, n, k, chosen)
            assert traffic_rot is not None, f"{name}_rotating_b: {source_rot}"
    # a summary of another configuration is not used
    t, why = bench.profiled_traffic("square8192", 8192, 8192, 8192, "q128x128_w2x2_s9o1")
    assert t is None and "not used" in why


def test_benchmark_table_rows_name_the_kernels_the_library_chooses():
    path = os.path.join(ROOT, "benchmarks", "mi355x.md")
    rows = [l for l in open(path).read().splitlines() if re.match(r"^\| \d+ \| \d+ \| \d+ \|", l)]
    from quadmul_amd.autotune import REFERENCE_SHAPES

    seen = set()
    for l in rows:
        cells = [c.strip() for c in l.strip("|").split("|")]
        m, n, k = int(cells[0]), int(cells[1]), int(cells[2])
        kernel = cells[-1]
        if (m, n, k) in seen:     # (the second table, timed through the bare seven-argument entry point)
            chosen = qm.config_name(qm.select_config_ex(m, n, k, workspace=False) & 0xFFFF)
        else:
            chosen = qm.config_name(qm.select_config(m, n, k) & 0xFFFF)
        seen.add((m, n, k))
        assert kernel == chosen, f"benchmarks/mi355x.md row {m}x{n}x{k} names {kernel}, the library chooses {chosen}: regenerate the table"
    assert seen == set(REFERENCE_SHAPES), "the table must cover the reference's 42 shapes (kernel.cu:343-384)"


def test_the_build_scans_for_scalar_operands_written_just_before_an_asm_load_or_store(tmp_path):
    """A memory instruction inside an asm statement that reads a scalar register fewer than
    five wait states after a vector instruction wrote it: quadmul_amd.build's scan finds it
    (the compiler keeps that distance for its own memory instructions only)."""
    from quadmul_amd.build import scalar_operand_hazards

    isa = tmp_path / "unit.s"
    isa.write_text("\n".join([
        "\tv_readlane_b32 s10, v193, 49",
        "\tv_readlane_b32 s11, v193, 50",
        "\t;;#ASMSTART",
        "\tglobal_load_lds_dwordx4 v156, s[10:11]",            # one wait state after the write: found
        "\t;;#ASMEND",
        "\tv_readlane_b32 s5, v1, 3",
        "\ts_nop 4",
        "\tglobal_store_dwordx4 v118, v[72:75], s[4:5]",      # five wait states: fine
        "\tv_readfirstlane_b32 s20, v7",
        "\tv_add_u32_e32 v1, v2, v3",
        "\ts_mov_b64 s[30:31], exec",
        "\tglobal_store_dwordx2 v118, v[72:73], s[20:21]",    # three: found
        "\ts_add_u32 s40, s2, s3",
        "\tglobal_store_dwordx4 v118, v[72:75], s[40:41]",    # written by a scalar instruction: fine
        "\tv_cmp_ne_u32_e64 s[50:51], 0, v0",
        "\tglobal_store_dwordx4 v1, v[2:5], off",             # no scalar operand
        ""]))
    found = scalar_operand_hazards(str(isa))
    assert [f[0] for f in found] == [4, 12], found
    assert "v_readlane_b32 s11" in found[0][1] and "v_readfirstlane_b32 s20" in found[1][1]
