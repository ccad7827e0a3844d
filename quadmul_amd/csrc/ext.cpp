// PyTorch-ROCm extension module `quadmul`: the drop-in for the reference's
// pybind11 module (extension.cpp:8-29) -- same module name (setup.py:8,11), same
// function gemm(a, b, c, m, n, k) -> None, same positional order (test.py:40).
// Host-only C++: tensors are unwrapped to device pointers and handed, with the
// current HIP stream of a's device (extension.cpp:23), to the C ABI in
// include/qm_abi.h.  No kernels and no HIP runtime calls live here.
//
// The argument checks the reference left commented out (extension.cpp:11-15) are
// live here; a non-zero status from the library is raised as RuntimeError.
#include <torch/extension.h>
#include <torch/library.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "qm_abi.h"

namespace {

void check_status(int status, const char *what)
{
    if (status == QM_OK) return;
    if (status == QM_ERR_LAUNCH)
        TORCH_CHECK(false, what, ": ", qm_status_string(status), " (hipError_t ", qm_last_hip_error(), ")");
    TORCH_CHECK(false, what, ": ", qm_status_string(status));
}

bool is_byte(const torch::Tensor &t) { return t.scalar_type() == torch::kInt8 || t.scalar_type() == torch::kUInt8; }

void *stream_of(const torch::Tensor &t) { return static_cast<void *>(c10::hip::getCurrentHIPStream(t.get_device()).stream()); }

void check_operands(const torch::Tensor &a, const torch::Tensor &b, const torch::Tensor &c, int64_t m, int64_t n, int64_t k,
                    bool scaled = false)
{
    TORCH_CHECK(a.is_cuda() && b.is_cuda() && c.is_cuda(), "quadmul.gemm: a, b and c must be GPU tensors");
    TORCH_CHECK(a.device() == b.device() && a.device() == c.device(), "quadmul.gemm: all tensors must be on the same device");
    // pack_b yields int8 (test.py:14); the reference only ever looks at data_ptr().
    TORCH_CHECK(is_byte(a) && is_byte(b), "quadmul.gemm: a and b must be int8 or uint8 (packed int4)");
    if (scaled) {
        TORCH_CHECK(c.scalar_type() == torch::kFloat16 || c.scalar_type() == torch::kBFloat16, "quadmul.gemm_scaled: d must be float16 or bfloat16");
    } else {
        TORCH_CHECK(c.scalar_type() == torch::kInt32, "quadmul.gemm: c must be int32");
    }
    TORCH_CHECK(a.is_contiguous() && b.is_contiguous() && c.is_contiguous(), "quadmul.gemm: all tensors must be contiguous");
    TORCH_CHECK(m >= 0 && n >= 0 && k >= 0 && k % 2 == 0, "quadmul.gemm: m, n, k must be >= 0 and k even");
    TORCH_CHECK(m <= INT32_MAX && n <= INT32_MAX && k <= INT32_MAX, "quadmul.gemm: m, n, k must fit in int32");
    TORCH_CHECK(a.numel() == m * (k / 2), "quadmul.gemm: a must hold m*k/2 bytes, got ", a.numel());
    TORCH_CHECK(b.numel() == n * (k / 2), "quadmul.gemm: b must hold n*k/2 bytes, got ", b.numel());
    TORCH_CHECK(c.numel() == m * n, "quadmul.gemm: c must hold m*n int32, got ", c.numel());
}

// The workspace of a call that splits K (few output tiles, long K), from torch's caching
// allocator: stream-ordered, so calls on different streams never share one, and legal under
// graph capture.  An undefined tensor when the shape does not split.
int ptr_alignment(const torch::Tensor &a, const torch::Tensor &b)
{
    const uintptr_t x = reinterpret_cast<uintptr_t>(a.data_ptr()) | reinterpret_cast<uintptr_t>(b.data_ptr());
    if (x == 0) return 4096;
    const uintptr_t low = x & (~x + 1);
    return low > 4096 ? 4096 : (int)low;
}

torch::Tensor workspace_for(const torch::Tensor &a, const torch::Tensor &b, int64_t m, int64_t n, int64_t k, int cfg, bool scaled)
{
    const size_t need = qm_gemm_workspace_bytes((int)m, (int)n, (int)k, ptr_alignment(a, b), cfg, scaled ? 1 : 0);
    if (need == 0) return torch::Tensor();
    return torch::empty({(int64_t)need}, a.options().dtype(torch::kUInt8));
}

void gemm(torch::Tensor a, torch::Tensor b, torch::Tensor c, int64_t m, int64_t n, int64_t k)
{
    check_operands(a, b, c, m, n, k);
    c10::OptionalDeviceGuard guard(a.device());
    const torch::Tensor ws = workspace_for(a, b, m, n, k, QM_CFG_AUTO, false);
    check_status(qm_gemm_i4_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), (int)m, (int)n, (int)k, stream_of(a), QM_CFG_AUTO,
                               ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0),
                 "quadmul.gemm");
}

// The GEMM with the dequantising epilogue fused in (no counterpart in the reference's code;
// its README.md:7 names the idea): d = round(((float)c * row_scale[m]) * col_scale[n]), d
// float16 or bfloat16, the scales float32 vectors on a's device (an undefined tensor = ones).
void check_scale(const c10::optional<torch::Tensor> &s, const torch::Tensor &a, int64_t count, const char *what)
{
    if (!s.has_value()) return;
    TORCH_CHECK(s->is_cuda() && s->device() == a.device() && s->scalar_type() == torch::kFloat32 && s->is_contiguous() && s->numel() == count,
                "quadmul.gemm_scaled: ", what, " must be a contiguous float32 vector of ", count, " elements on a's device");
}

void gemm_scaled(torch::Tensor a, torch::Tensor b, torch::Tensor d, int64_t m, int64_t n, int64_t k,
                 c10::optional<torch::Tensor> row_scale, c10::optional<torch::Tensor> col_scale)
{
    check_operands(a, b, d, m, n, k, true);
    check_scale(row_scale, a, m, "row_scale");
    check_scale(col_scale, a, n, "col_scale");
    c10::OptionalDeviceGuard guard(a.device());
    const int out = d.scalar_type() == torch::kFloat16 ? QM_OUT_F16 : QM_OUT_BF16;
    const torch::Tensor ws = workspace_for(a, b, m, n, k, QM_CFG_AUTO, true);
    check_status(qm_gemm_i4_scaled_ws(a.data_ptr(), b.data_ptr(), d.data_ptr(), (int)m, (int)n, (int)k,
                                      row_scale.has_value() ? row_scale->data_ptr<float>() : nullptr,
                                      col_scale.has_value() ? col_scale->data_ptr<float>() : nullptr, out, stream_of(a), QM_CFG_AUTO,
                                      ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0),
                 "quadmul.gemm_scaled");
}

void gemm_cfg(torch::Tensor a, torch::Tensor b, torch::Tensor c, int64_t m, int64_t n, int64_t k, int64_t cfg)
{
    check_operands(a, b, c, m, n, k);
    c10::OptionalDeviceGuard guard(a.device());
    const torch::Tensor ws = workspace_for(a, b, m, n, k, (int)cfg, false);
    check_status(qm_gemm_i4_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), (int)m, (int)n, (int)k, stream_of(a), (int)cfg,
                               ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0),
                 "quadmul.gemm_cfg");
}

// Device-side pack_b (test.py:6-15): [rows, K] int8 -> [rows, K/2] int8.
torch::Tensor pack(torch::Tensor values)
{
    TORCH_CHECK(values.is_cuda() && values.scalar_type() == torch::kInt8 && values.dim() == 2, "quadmul.pack: expects a 2-D int8 GPU tensor");
    TORCH_CHECK(values.size(1) % 2 == 0, "quadmul.pack: K must be even");
    auto v = values.contiguous();
    c10::OptionalDeviceGuard guard(v.device());
    auto out = torch::empty({v.size(0), v.size(1) / 2}, v.options());
    check_status(qm_pack_i4(v.data_ptr(), out.data_ptr(), (int)v.size(0), (int)v.size(1), stream_of(v)), "quadmul.pack");
    return out;
}

// Per-row symmetric int4 quantisation fused with the packing (no counterpart in the
// reference beyond pack_b's packing half): [rows, K] fp16 / bf16 / fp32 -> ([rows, K/2]
// int8, [rows] float32 scales = amax / 7, the row_scale of gemm_scaled).
std::tuple<torch::Tensor, torch::Tensor> quantize_pack(torch::Tensor x)
{
    TORCH_CHECK(x.is_cuda() && x.dim() == 2, "quadmul.quantize_pack: expects a 2-D GPU tensor");
    const auto t = x.scalar_type();
    TORCH_CHECK(t == torch::kFloat16 || t == torch::kBFloat16 || t == torch::kFloat32, "quadmul.quantize_pack: x must be float16, bfloat16 or float32");
    TORCH_CHECK(x.size(1) % 2 == 0, "quadmul.quantize_pack: K must be even");
    auto v = x.contiguous();
    c10::OptionalDeviceGuard guard(v.device());
    auto packed = torch::empty({v.size(0), v.size(1) / 2}, v.options().dtype(torch::kInt8));
    auto scales = torch::empty({v.size(0)}, v.options().dtype(torch::kFloat32));
    const int in = t == torch::kFloat16 ? QM_IN_F16 : (t == torch::kBFloat16 ? QM_IN_BF16 : QM_IN_F32);
    check_status(qm_quantize_pack_i4(v.data_ptr(), in, packed.data_ptr(), scales.data_ptr<float>(), (int)v.size(0), (int)v.size(1), stream_of(v)),
                 "quadmul.quantize_pack");
    return {packed, scales};
}

// Device-side unpack_int4_matrix (kernel.cu:389-408): [rows, K/2] bytes -> [rows, K] int8.
torch::Tensor unpack(torch::Tensor packed)
{
    TORCH_CHECK(packed.is_cuda() && is_byte(packed) && packed.dim() == 2, "quadmul.unpack: expects a 2-D int8/uint8 GPU tensor");
    auto p = packed.contiguous();
    c10::OptionalDeviceGuard guard(p.device());
    auto out = torch::empty({p.size(0), p.size(1) * 2}, p.options().dtype(torch::kInt8));
    check_status(qm_unpack_i4(p.data_ptr(), out.data_ptr(), (int)p.size(0), (int)p.size(1) * 2, stream_of(p)), "quadmul.unpack");
    return out;
}

// Dispatcher-visible form of the same op (schema + mutation annotation), so that callers
// under torch.compile / export can keep `torch.ops.quadmul.gemm(a, b, c, m, n, k)` in the
// graph.  The reference has only the pybind function (extension.cpp:26-29), which a tracer
// cannot see through.  c is written in place; nothing is returned.
void gemm_meta(const torch::Tensor &, const torch::Tensor &, torch::Tensor &, int64_t, int64_t, int64_t) {}
void gemm_op(const torch::Tensor &a, const torch::Tensor &b, torch::Tensor &c, int64_t m, int64_t n, int64_t k) { gemm(a, b, c, m, n, k); }
void gemm_scaled_meta(const torch::Tensor &, const torch::Tensor &, torch::Tensor &, int64_t, int64_t, int64_t,
                      const c10::optional<torch::Tensor> &, const c10::optional<torch::Tensor> &) {}
void gemm_scaled_op(const torch::Tensor &a, const torch::Tensor &b, torch::Tensor &d, int64_t m, int64_t n, int64_t k,
                    const c10::optional<torch::Tensor> &row_scale, const c10::optional<torch::Tensor> &col_scale)
{
    gemm_scaled(a, b, d, m, n, k, row_scale, col_scale);
}

// quantize_pack returns new tensors: the Meta form only has to give their shapes and types
std::tuple<torch::Tensor, torch::Tensor> quantize_pack_meta(const torch::Tensor &x)
{
    TORCH_CHECK(x.dim() == 2 && x.size(1) % 2 == 0, "quadmul.quantize_pack: expects a 2-D tensor with even K");
    return {torch::empty({x.size(0), x.size(1) / 2}, x.options().dtype(torch::kInt8)), torch::empty({x.size(0)}, x.options().dtype(torch::kFloat32))};
}
std::tuple<torch::Tensor, torch::Tensor> quantize_pack_op(const torch::Tensor &x) { return quantize_pack(x); }

}  // namespace

TORCH_LIBRARY(quadmul, m)
{
    m.def("gemm(Tensor a, Tensor b, Tensor(c!) c, int m, int n, int k) -> ()");
    m.def("gemm_scaled(Tensor a, Tensor b, Tensor(d!) d, int m, int n, int k, Tensor? row_scale, Tensor? col_scale) -> ()");
    m.def("quantize_pack(Tensor x) -> (Tensor, Tensor)");
}
TORCH_LIBRARY_IMPL(quadmul, CUDA, m)
{
    m.impl("gemm", &gemm_op);
    m.impl("gemm_scaled", &gemm_scaled_op);
    m.impl("quantize_pack", &quantize_pack_op);
}
TORCH_LIBRARY_IMPL(quadmul, Meta, m)
{
    m.impl("gemm", &gemm_meta);
    m.impl("gemm_scaled", &gemm_scaled_meta);
    m.impl("quantize_pack", &quantize_pack_meta);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("gemm", &gemm, "Int4xInt4 Matrix Multiplication Kernel", py::arg("a"), py::arg("b"), py::arg("c"), py::arg("m"), py::arg("n"), py::arg("k"));
    m.def("gemm_scaled", &gemm_scaled, "Int4xInt4 GEMM with per-row and per-column fp32 scales, fp16 / bf16 output", py::arg("a"), py::arg("b"),
          py::arg("d"), py::arg("m"), py::arg("n"), py::arg("k"), py::arg("row_scale") = py::none(), py::arg("col_scale") = py::none());
    m.def("gemm_cfg", &gemm_cfg, "gemm with an explicit kernel configuration id (autotuning)");
    m.def("pack", &pack, "Pack a [rows, K] int8 tensor of int4 values into [rows, K/2] bytes on the GPU");
    m.def("quantize_pack", &quantize_pack, "Per-row symmetric int4 quantisation of a [rows, K] float tensor, packed; returns (packed, scales)");
    m.def("unpack", &unpack, "Unpack [rows, K/2] bytes into a [rows, K] int8 tensor on the GPU");
    m.def("num_configs", &qm_num_configs);
    m.def("config_name", [](int cfg) { const char *s = qm_config_name(cfg); return std::string(s ? s : ""); });
    m.def("select_config", &qm_select_config);
    m.def("version", []() { return std::string(qm_version()); });
}
