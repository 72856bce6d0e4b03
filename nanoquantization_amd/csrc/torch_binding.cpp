// PyTorch-ROCm operator binding over the C ABI of libawq_hip.so (include/awq_hip.h).
//
// No kernels here: every operator checks its arguments the way the reference's Python entry points do
// (nanoquantization/layers/gemm.py:126-180 awq_dequantize, :329-379 awq_gemm, :552-567 WQLinear_GEMM.forward),
// allocates the output with torch, and calls the C entry point on torch's current HIP stream -- where the
// reference's Triton launches go (layers/gemm.py:363-377).  Registered as
//   torch.ops.nanoquantization_amd.awq_dequantize(qweight, qscales, qzeros) -> Tensor [K, N]
//   torch.ops.nanoquantization_amd.awq_linear(x, qweight, qscales, qzeros, bias?) -> Tensor [M, N]
//   torch.ops.nanoquantization_amd.awq_linear_swiglu(x, qweight, qscales, qzeros) -> Tensor [M, N / 2]
// with Meta kernels (shapes only), so the operators are visible to the dispatcher and to tracing.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/awq_hip.h"

namespace {

// PyTorch-ROCm labels HIP tensors and streams with the device type "cuda"; these are the HIP guard and stream
// getters for that labelling.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
hipStream_t current_stream(c10::DeviceIndex index) {
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(index).stream();
}

struct Packed {
    int64_t K, N, g;
    int dtype;
};

Packed check_packed(const at::Tensor& qweight, const at::Tensor& qscales, const at::Tensor& qzeros) {
    TORCH_CHECK(qweight.dim() == 2 && qscales.dim() == 2 && qzeros.dim() == 2,
                "qweight, qscales and qzeros must be 2-D");
    TORCH_CHECK(qweight.scalar_type() == at::kInt && qzeros.scalar_type() == at::kInt,
                "qweight and qzeros must be int32");
    TORCH_CHECK(qscales.scalar_type() == at::kHalf || qscales.scalar_type() == at::kBFloat16,
                "qscales dtype must be float16 or bfloat16, got ", qscales.scalar_type());
    Packed p;
    p.K = qweight.size(0);
    p.N = qscales.size(1);
    TORCH_CHECK(p.K > 0 && p.N > 0 && qscales.size(0) > 0, "empty packed weight");
    p.g = p.K / qscales.size(0);
    TORCH_CHECK(qweight.size(1) * 8 == p.N, "qweight must be [K, N/8]");
    TORCH_CHECK(qscales.size(0) * p.g == p.K, "qscales must be [K/g, N]");
    TORCH_CHECK(qzeros.size(0) == qscales.size(0) && qzeros.size(1) * 8 == p.N, "qzeros must be [K/g, N/8]");
    TORCH_CHECK(p.g == 32 || p.g == 64 || p.g == 128 || p.g == p.K, "unsupported group size ", p.g);
    p.dtype = qscales.scalar_type() == at::kHalf ? AWQ_F16 : AWQ_BF16;
    return p;
}

void check_device(const at::Tensor& ref, std::initializer_list<const at::Tensor*> others) {
    TORCH_CHECK(ref.is_cuda(), "AWQ kernels run on a HIP device only (tensor is on ", ref.device(),
                "); there is no CPU fallback");
    for (const at::Tensor* t : others)
        TORCH_CHECK(t->device() == ref.device(), "tensors on different devices: ", t->device(), " vs ", ref.device());
}

void check_status(int status, const char* entry) {
    TORCH_CHECK(status == AWQ_OK, "libawq_hip: ", entry, " failed (status ", status, "): ", awq_hip_last_error());
}

// One zero-filled split-K workspace per (device, stream).  The kernels leave it zeroed and calls on one stream are
// ordered, so every layer shares it.  A workspace is never freed: a HIP graph captured while it was current keeps
// its address, so a larger request retires the old tensor instead of releasing it.
struct WsKey {
    int device;
    void* stream;
    bool operator==(const WsKey& o) const { return device == o.device && stream == o.stream; }
};
struct WsHash {
    size_t operator()(const WsKey& k) const { return std::hash<void*>()(k.stream) ^ (size_t)k.device * 0x9E3779B97F4A7C15ull; }
};
std::mutex g_ws_mutex;
std::unordered_map<WsKey, at::Tensor, WsHash> g_ws;
std::vector<at::Tensor> g_ws_retired;

at::Tensor workspace(const at::Device& dev, void* stream, size_t nbytes) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    const WsKey key{dev.index(), stream};
    auto it = g_ws.find(key);
    if (it != g_ws.end() && (size_t)it->second.numel() >= nbytes) return it->second;
    if (it != g_ws.end()) g_ws_retired.push_back(it->second);
    const int64_t size = (int64_t)std::max<size_t>(nbytes, (size_t)8 << 20);
    at::Tensor ws = at::zeros({size}, at::TensorOptions().dtype(at::kByte).device(dev));
    g_ws[key] = ws;
    return ws;
}

at::Tensor awq_dequantize_op(const at::Tensor& qweight, const at::Tensor& qscales, const at::Tensor& qzeros) {
    const Packed p = check_packed(qweight, qscales, qzeros);
    check_device(qweight, {&qscales, &qzeros});
    const DeviceGuard guard(qweight.device());
    const at::Tensor qw = qweight.contiguous(), qs = qscales.contiguous(), qz = qzeros.contiguous();
    at::Tensor out = at::empty({p.K, p.N}, qs.options());
    hipStream_t stream = current_stream(qw.device().index());
    check_status(awq_dequantize(qw.data_ptr<int32_t>(), qs.data_ptr(), qz.data_ptr<int32_t>(), out.data_ptr(), p.K,
                                p.N, p.g, p.dtype, stream),
                 "awq_dequantize");
    return out;
}

at::Tensor awq_dequantize_meta(const at::Tensor& qweight, const at::Tensor& qscales, const at::Tensor& qzeros) {
    return at::empty({qweight.size(0), qscales.size(1)}, qscales.options());
}

using LinearEntry = int (*)(const void*, const int32_t*, const void*, const int32_t*, const void*, void*, int64_t,
                            int64_t, int64_t, int64_t, int, void*, size_t, void*);

at::Tensor awq_linear_op(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qscales,
                         const at::Tensor& qzeros, const c10::optional<at::Tensor>& bias) {
    const Packed p = check_packed(qweight, qscales, qzeros);
    TORCH_CHECK(x.dim() == 2 && x.size(1) == p.K, "x must be [M, ", p.K, "], got ", x.sizes());
    check_device(x, {&qweight, &qscales, &qzeros});
    const DeviceGuard guard(x.device());
    const at::ScalarType dt = qscales.scalar_type();
    // the reference casts x to the output dtype on load (layers/gemm.py:259)
    const at::Tensor xc = (x.scalar_type() == dt ? x : x.to(dt)).contiguous();
    const at::Tensor qw = qweight.contiguous(), qs = qscales.contiguous(), qz = qzeros.contiguous();
    at::Tensor b;
    if (bias.has_value() && bias->defined()) {
        TORCH_CHECK(bias->numel() == p.N, "bias must have ", p.N, " elements");
        b = bias->to(x.device(), dt).contiguous();
    }
    const int64_t M = xc.size(0);
    at::Tensor out = at::empty({M, p.N}, qs.options());
    if (M == 0) return out;
    hipStream_t stream = current_stream(x.device().index());
    const size_t nbytes = awq_linear_workspace_bytes(M, p.N, p.K);
    at::Tensor ws;
    if (nbytes) ws = workspace(x.device(), stream, nbytes);
    check_status(awq_linear(xc.data_ptr(), qw.data_ptr<int32_t>(), qs.data_ptr(), qz.data_ptr<int32_t>(),
                            b.defined() ? b.data_ptr() : nullptr, out.data_ptr(), M, p.N, p.K, p.g, p.dtype,
                            nbytes ? ws.data_ptr() : nullptr, nbytes ? (size_t)ws.numel() : 0, stream),
                 "awq_linear");
    return out;
}

at::Tensor awq_linear_meta(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qscales,
                           const at::Tensor& qzeros, const c10::optional<at::Tensor>& bias) {
    return at::empty({x.size(0), qscales.size(1)}, qscales.options());
}

at::Tensor awq_linear_swiglu_op(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qscales,
                                const at::Tensor& qzeros) {
    const Packed p = check_packed(qweight, qscales, qzeros);
    TORCH_CHECK(x.dim() == 2 && x.size(1) == p.K, "x must be [M, ", p.K, "], got ", x.sizes());
    TORCH_CHECK(p.N % 16 == 0, "gate|up interleaved by words needs N % 16 == 0");
    check_device(x, {&qweight, &qscales, &qzeros});
    const DeviceGuard guard(x.device());
    const at::ScalarType dt = qscales.scalar_type();
    const at::Tensor xc = (x.scalar_type() == dt ? x : x.to(dt)).contiguous();
    const at::Tensor qw = qweight.contiguous(), qs = qscales.contiguous(), qz = qzeros.contiguous();
    const int64_t M = xc.size(0);
    at::Tensor out = at::empty({M, p.N / 2}, qs.options());
    if (M == 0) return out;
    hipStream_t stream = current_stream(x.device().index());
    const size_t nbytes = awq_linear_swiglu_workspace_bytes(M, p.N, p.K);
    at::Tensor ws;
    if (nbytes) ws = workspace(x.device(), stream, nbytes);
    check_status(awq_linear_swiglu(xc.data_ptr(), qw.data_ptr<int32_t>(), qs.data_ptr(), qz.data_ptr<int32_t>(),
                                   out.data_ptr(), M, p.N, p.K, p.g, p.dtype, nbytes ? ws.data_ptr() : nullptr,
                                   nbytes ? (size_t)ws.numel() : 0, stream),
                 "awq_linear_swiglu");
    return out;
}

at::Tensor awq_linear_swiglu_meta(const at::Tensor& x, const at::Tensor& qweight, const at::Tensor& qscales,
                                  const at::Tensor& qzeros) {
    return at::empty({x.size(0), qscales.size(1) / 2}, qscales.options());
}

}  // namespace

TORCH_LIBRARY(nanoquantization_amd, m) {
    m.def("awq_dequantize(Tensor qweight, Tensor qscales, Tensor qzeros) -> Tensor");
    m.def("awq_linear(Tensor x, Tensor qweight, Tensor qscales, Tensor qzeros, Tensor? bias=None) -> Tensor");
    m.def("awq_linear_swiglu(Tensor x, Tensor qweight, Tensor qscales, Tensor qzeros) -> Tensor");
}

TORCH_LIBRARY_IMPL(nanoquantization_amd, CUDA, m) {   // the dispatch key of HIP tensors in PyTorch-ROCm
    m.impl("awq_dequantize", &awq_dequantize_op);
    m.impl("awq_linear", &awq_linear_op);
    m.impl("awq_linear_swiglu", &awq_linear_swiglu_op);
}

TORCH_LIBRARY_IMPL(nanoquantization_amd, Meta, m) {
    m.impl("awq_dequantize", &awq_dequantize_meta);
    m.impl("awq_linear", &awq_linear_meta);
    m.impl("awq_linear_swiglu", &awq_linear_swiglu_meta);
}
