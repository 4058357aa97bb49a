// PyTorch extension over the C ABI (include/fp6mi.h): the per-call path of the Python package in C++, the part
// fp6_llm/csrc/pybind.cpp:6-16 and the torch wrappers of fp6_llm/csrc/fp6_linear.cu:161-201,269-313 play in the reference.
// A plain host translation unit: it touches torch only for tensors, the current stream and the device guard, and hands
// raw pointers to libfp6mi.so.  The Python package uses it when it is built and falls back to its ctypes binding of the
// same C ABI otherwise; both launch the same kernels.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <string>
#include <utility>

#include "fp6mi.h"
#include "fp6_linear_torch.h"

namespace {

[[noreturn]] void bad(const std::string &msg) { throw pybind11::value_error(msg); }

std::mutex                                         g_ws_mutex;
std::map<std::pair<int, void *>, at::Tensor>       g_workspaces; // (device, stream) -> float32 tensor, grown on demand

at::Tensor workspace_for(const at::Device &dev, void *stream, int64_t floats)
{
    // Under stream capture the memory belongs to the graph being recorded: this call gets a tensor of its own (the graph keeps
    // the memory for its replays) and nothing is remembered, or a later eager call would share scratch with those replays.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capture) == hipSuccess && capture != hipStreamCaptureStatusNone)
        return at::empty({ floats }, at::TensorOptions().dtype(at::kFloat).device(dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto                        key = std::make_pair((int)dev.index(), stream);
    auto                        it = g_workspaces.find(key);
    if (it == g_workspaces.end() || it->second.numel() < floats) {
        at::Tensor t = at::empty({ floats }, at::TensorOptions().dtype(at::kFloat).device(dev));
        g_workspaces[key] = t;
        return t;
    }
    return it->second;
}

// out[B, OC] = in_feats[B, IC] @ dequant(W)^T with W in the native layout, enqueued on the current stream of in_feats' device.
at::Tensor linear_forward_native(int64_t E, int64_t Mb, const at::Tensor &in_feats, const at::Tensor &native_weight, const at::Tensor &scales,
                                 int64_t OC, int64_t splitK, const c10::optional<at::Tensor> &out_opt, const c10::optional<at::Tensor> &ws_opt,
                                 const c10::optional<at::Tensor> &gexp_opt)
{
    const bool known = (E == 3 && Mb == 2) || (E == 2 && Mb >= 1 && Mb <= 3);
    if (!known) bad("unsupported format: EXPONENT=" + std::to_string(E) + ", MANTISSA=" + std::to_string(Mb) + " (only e3m2, e2m2, e2m3 and e2m1)");
    if (in_feats.scalar_type() != at::kHalf || in_feats.dim() != 2) bad("in_feats must be a 2-D float16 tensor [B, IC]");
    if (!in_feats.is_cuda()) bad("in_feats must be on the GPU");
    const at::Device dev = in_feats.device();
    if (native_weight.device() != dev || scales.device() != dev) bad("in_feats, weights and scales must be on the same GPU");
    if (scales.scalar_type() != at::kHalf || scales.numel() != OC) bad("scales must be float16 [OC]");
    const int64_t B = in_feats.size(0), IC = in_feats.size(1);
    if (OC % 256 != 0 || IC % 64 != 0 || B < 1) bad("need OC % 256 == 0, IC % 64 == 0, B >= 1");
    const int64_t want = (int64_t)fp6mi_native_bytes((int)E, (int)Mb, (size_t)OC, (size_t)IC);
    if ((int64_t)native_weight.numel() * (int64_t)native_weight.element_size() != want) bad("native_weight has the wrong size for OC and IC");
    if (splitK < 1) bad("splitK must be >= 1");
    if (!native_weight.is_contiguous()) bad("native_weight must be contiguous");
    at::Tensor x = in_feats.is_contiguous() ? in_feats : in_feats.contiguous();
    at::Tensor sc = scales.is_contiguous() ? scales : scales.contiguous();
    at::Tensor out;
    if (out_opt.has_value()) {
        out = *out_opt;
        if (out.dim() != 2 || out.size(0) != B || out.size(1) != OC || out.scalar_type() != at::kHalf || !out.is_contiguous() || out.device() != dev)
            bad("out must be a contiguous float16 [B, OC] tensor on the same GPU");
    }
    c10::hip::HIPGuard guard(dev.index());
    if (!out_opt.has_value()) out = at::empty({ B, OC }, at::TensorOptions().dtype(at::kHalf).device(dev));
    void  *stream = c10::hip::getCurrentHIPStream(dev.index()).stream();
    float *ws_ptr = nullptr;
    at::Tensor ws;
    if (splitK > 1) {
        const int64_t need = splitK * B * OC;
        if (ws_opt.has_value()) {
            ws = *ws_opt;
            if (ws.scalar_type() != at::kFloat || ws.numel() < need || ws.device() != dev || !ws.is_contiguous())
                bad("workspace must be a contiguous float32 GPU tensor with at least splitK*B*OC elements");
        } else {
            ws = workspace_for(dev, stream, need);
        }
        ws_ptr = ws.data_ptr<float>();
    }
    int rc;
    if (gexp_opt.has_value()) { // per-group exponents in the kernels' own order (fp6mi_pack_group_exps)
        const at::Tensor &g = *gexp_opt;
        if (g.scalar_type() != at::kByte || g.device() != dev || !g.is_contiguous() || g.numel() != (int64_t)fp6mi_group_exps_bytes((size_t)OC, (size_t)IC))
            bad("group_exps must be the contiguous uint8 tensor of pack_group_exps(exps, OC, IC) on the weights' GPU");
        rc = fp6mi_linear_native_grouped((int)E, (int)Mb, stream, native_weight.data_ptr(), sc.data_ptr(), g.data_ptr(), x.data_ptr(), out.data_ptr(),
                                         (size_t)OC, (size_t)B, (size_t)IC, ws_ptr, (int)splitK);
    } else {
        rc = fp6mi_linear_native((int)E, (int)Mb, stream, native_weight.data_ptr(), sc.data_ptr(), x.data_ptr(), out.data_ptr(), (size_t)OC, (size_t)B,
                                 (size_t)IC, ws_ptr, (int)splitK);
    }
    if (rc != 0) throw std::runtime_error(std::string("fp6mi_linear_native: ") + fp6mi_error_string(rc));
    return out;
}

void clear_workspaces()
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_workspaces.clear();
}

// ---- native twins of reference-layout GPU weights, for the reference-named C++ entry points below ----
// Keyed by the tensor's implementation object and remembered while that object is alive and unmodified (same storage address,
// same in-place version counter), like the Python package does for its callers.  A twin is published only once its relayout
// kernel has finished; a first use under stream capture converts into the graph's pool and is not remembered.
struct TwinEntry {
    c10::weak_intrusive_ptr<c10::TensorImpl> owner;
    uint32_t                                 version;
    void                                    *data;
    int                                      E, Mb;
    at::Tensor                               native;
};
std::mutex                                   g_twin_mutex;
std::map<c10::TensorImpl *, TwinEntry>       g_twin_cache;

void check_format(int64_t E, int64_t Mb)
{
    const bool known = (E == 3 && Mb == 2) || (E == 2 && Mb >= 1 && Mb <= 3);
    if (!known) bad("unsupported format: EXPONENT=" + std::to_string(E) + ", MANTISSA=" + std::to_string(Mb) + " (only e3m2, e2m2, e2m3 and e2m1)");
}

// [OC, IC] of an int32 [OC, IC/32*x] weight tensor (raw or prepacked: same shape)
std::pair<int64_t, int64_t> weight_shape(const at::Tensor &t, int64_t E, int64_t Mb, const char *name)
{
    check_format(E, Mb);
    const int64_t x = 1 + E + Mb;
    if (t.scalar_type() != at::kInt || t.dim() != 2) bad(std::string(name) + " must be a 2-D int32 tensor [OC, IC/32*" + std::to_string(x) + "]");
    if (t.size(1) % x != 0) bad(std::string(name) + ".size(1) is not a multiple of " + std::to_string(x));
    return { t.size(0), t.size(1) / x * 32 };
}

at::Tensor native_twin_of(const at::Tensor &weights, int64_t E, int64_t Mb, int64_t OC, int64_t IC)
{
    c10::TensorImpl *impl = weights.unsafeGetTensorImpl();
    {
        std::lock_guard<std::mutex> lock(g_twin_mutex);
        auto it = g_twin_cache.find(impl);
        if (it != g_twin_cache.end()) {
            TwinEntry &e = it->second;
            auto       alive = e.owner.lock();
            if (alive && alive.get() == impl && e.version == weights._version() && e.data == weights.data_ptr() && e.E == E && e.Mb == Mb) return e.native;
            g_twin_cache.erase(it);
        }
        if (g_twin_cache.size() > 4096) // drop the entries of tensors that are gone
            for (auto i = g_twin_cache.begin(); i != g_twin_cache.end();) i = i->second.owner.expired() ? g_twin_cache.erase(i) : std::next(i);
    }
    const at::Device dev = weights.device();
    c10::hip::HIPGuard guard(dev.index());
    auto               hip_stream = c10::hip::getCurrentHIPStream(dev.index());
    at::Tensor native = at::empty({ (int64_t)(fp6mi_native_bytes((int)E, (int)Mb, (size_t)OC, (size_t)IC) / 4) }, at::TensorOptions().dtype(at::kInt).device(dev));
    int        rc = fp6mi_relayout_ref_to_native_gpu((int)E, (int)Mb, hip_stream.stream(), native.data_ptr(), weights.data_ptr(), (size_t)OC, (size_t)IC);
    if (rc != 0) throw std::runtime_error(std::string("fp6mi_relayout_ref_to_native_gpu: ") + fp6mi_error_string(rc));
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(hip_stream.stream(), &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return native; // recorded, not run: nothing to remember
    hip_stream.synchronize();
    std::lock_guard<std::mutex> lock(g_twin_mutex);
    g_twin_cache.erase(impl);
    g_twin_cache.emplace(impl, TwinEntry{ c10::weak_intrusive_ptr<c10::TensorImpl>(weights.getIntrusivePtr()), weights._version(), weights.data_ptr(), (int)E, (int)Mb, native });
    return native;
}

} // namespace

// ------------------------------------------------------------------------------------------------ the reference's C++ names
// torch::Tensor entry points with the names, argument order and shapes of fp6_llm/csrc/fp6_linear.cuh:50-90, for C++ callers
// that link this extension (declared in fp6_linear_torch.h).  Where the reference asserts or exits these throw.

// fp6_llm/csrc/fp6_linear.cu:323-341 (weight_matrix_prepacking_fp_eXmY_cpu): raw int32 CPU [OC, IC/32*x] -> the reference's prepacked layout
torch::Tensor weight_matrix_prepacking_fp_eXmY_cpu(int EXPONENT, int MANTISSA, torch::Tensor fpx_tensor)
{
    auto [OC, IC] = weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor");
    if (OC % 256 != 0 || IC % 64 != 0) bad("weight_prepacking: need OC % 256 == 0 and IC % 64 == 0");
    if (!fpx_tensor.is_cpu()) bad("fpx_tensor must be a CPU tensor");
    at::Tensor src = fpx_tensor.contiguous(), out = at::empty_like(src);
    int        rc = fp6mi_prepack_ref(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), (size_t)OC, (size_t)IC);
    if (rc != 0) throw std::runtime_error(std::string("fp6mi_prepack_ref: ") + fp6mi_error_string(rc));
    return out;
}
// fp6_llm/csrc/fp6_linear.cu:211-223
torch::Tensor weight_matrix_prepacking_cpu(torch::Tensor fp6_tensor) { return weight_matrix_prepacking_fp_eXmY_cpu(3, 2, fp6_tensor); }

// fp6_llm/csrc/fp6_linear.cu:352-375 (weight_matrix_dequant_fp_eXmY_cpu): RAW weights + fp16 [OC] scales -> fp16 [OC, IC]
torch::Tensor weight_matrix_dequant_fp_eXmY_cpu(int EXPONENT, int MANTISSA, torch::Tensor fpx_tensor, torch::Tensor fp16_scale)
{
    auto [OC, IC] = weight_shape(fpx_tensor, EXPONENT, MANTISSA, "fpx_tensor");
    if (fp16_scale.scalar_type() != at::kHalf || fp16_scale.dim() != 1 || fp16_scale.size(0) != OC) bad("fp16_scale must be a float16 tensor of shape [OC]");
    if (!fpx_tensor.is_cpu() || !fp16_scale.is_cpu()) bad("fpx_tensor and fp16_scale must be CPU tensors");
    at::Tensor src = fpx_tensor.contiguous(), sc = fp16_scale.contiguous();
    at::Tensor out = at::empty({ OC, IC }, at::TensorOptions().dtype(at::kHalf));
    int        rc = fp6mi_dequant(EXPONENT, MANTISSA, out.data_ptr(), src.data_ptr(), (size_t)OC, (size_t)IC, sc.data_ptr());
    if (rc != 0) throw std::runtime_error(std::string("fp6mi_dequant: ") + fp6mi_error_string(rc));
    return out;
}
// fp6_llm/csrc/fp6_linear.cu:234-251
torch::Tensor weight_matrix_dequant_cpu(torch::Tensor fp6_tensor, torch::Tensor fp16_scale) { return weight_matrix_dequant_fp_eXmY_cpu(3, 2, fp6_tensor, fp16_scale); }

// fp6_llm/csrc/fp6_linear.cu:269-313 (fp_eXmY_linear_forward_cuda): _weights is the REFERENCE prepacked layout on the GPU; its
// native-layout twin is made by one relayout kernel on first use and kept while the tensor lives
torch::Tensor fp_eXmY_linear_forward_cuda(int EXPONENT, int MANTISSA, torch::Tensor _in_feats, torch::Tensor _weights, torch::Tensor _scales, int splitK)
{
    auto [OC, IC] = weight_shape(_weights, EXPONENT, MANTISSA, "weights");
    if (!_weights.is_cuda()) bad("weights must be on the GPU");
    if (!_weights.is_contiguous()) bad("weights must be contiguous");
    if (_in_feats.dim() != 2 || _in_feats.size(1) != IC) bad("in_feats must be [B, IC] with the weights' IC");
    if (OC % 256 != 0 || IC % 64 != 0) bad("need OC % 256 == 0, IC % 64 == 0");
    at::Tensor native = native_twin_of(_weights, EXPONENT, MANTISSA, OC, IC);
    return linear_forward_native(EXPONENT, MANTISSA, _in_feats, native, _scales, OC, splitK, c10::nullopt, c10::nullopt, c10::nullopt);
}
// fp6_llm/csrc/fp6_linear.cu:161-201
torch::Tensor fp6_linear_forward_cuda(torch::Tensor _in_feats, torch::Tensor _weights, torch::Tensor _scales, int splitK)
{
    return fp_eXmY_linear_forward_cuda(3, 2, _in_feats, _weights, _scales, splitK);
}

namespace {
void clear_twins()
{
    std::lock_guard<std::mutex> lock(g_twin_mutex);
    g_twin_cache.clear();
}
} // namespace

PYBIND11_MODULE(_fp6mi_torch, m)
{
    m.doc() = "torch tensors -> fp6mi C ABI";
    m.def("linear_forward_native", &linear_forward_native, pybind11::arg("EXPONENT"), pybind11::arg("MANTISSA"), pybind11::arg("in_feats"),
          pybind11::arg("native_weight"), pybind11::arg("scales"), pybind11::arg("OC"), pybind11::arg("splitK") = 1, pybind11::arg("out") = pybind11::none(),
          pybind11::arg("workspace") = pybind11::none(), pybind11::arg("group_exps") = pybind11::none());
    m.def("clear_workspaces", &clear_workspaces);
    m.def("clear_twins", &clear_twins);
    // the reference's bindings, name for name (fp6_llm/csrc/pybind.cpp:8-15)
    m.def("linear_forward_cuda", &fp6_linear_forward_cuda, "Computes FP6-FP16 GEMM.", pybind11::arg("in_feats"), pybind11::arg("weights"),
          pybind11::arg("scales"), pybind11::arg("splitK") = 1);
    m.def("weight_prepacking_cpu", &weight_matrix_prepacking_cpu, "Weight prepacking.");
    m.def("weight_dequant_cpu", &weight_matrix_dequant_cpu, "Dequantize weight from fp6 to fp16.");
    m.def("linear_forward_eXmY_cuda", &fp_eXmY_linear_forward_cuda, "Computes FPx-FP16 GEMM.", pybind11::arg("EXPONENT"), pybind11::arg("MANTISSA"),
          pybind11::arg("in_feats"), pybind11::arg("weights"), pybind11::arg("scales"), pybind11::arg("splitK") = 1);
    m.def("weight_prepacking_eXmY_cpu", &weight_matrix_prepacking_fp_eXmY_cpu, "FPx Weight prepacking.");
    m.def("weight_dequant_eXmY_cpu", &weight_matrix_dequant_fp_eXmY_cpu, "Dequantize weight from fpx to fp16.");
}
