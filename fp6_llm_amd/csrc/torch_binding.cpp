// PyTorch extension over the C ABI (include/fp6mi.h): the per-call path of the Python package in C++, the part
// fp6_llm/csrc/pybind.cpp:6-16 and the torch wrappers of fp6_llm/csrc/fp6_linear.cu:161-201,269-313 play in the reference.
// A plain host translation unit: it touches torch only for tensors, the current stream and the device guard, and hands
// raw pointers to libfp6mi.so.  The Python package uses it when it is built and falls back to its ctypes binding of the
// same C ABI otherwise; both launch the same kernels.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <map>
#include <mutex>
#include <string>
#include <utility>

#include "fp6mi.h"

namespace {

[[noreturn]] void bad(const std::string &msg) { throw pybind11::value_error(msg); }

std::mutex                                         g_ws_mutex;
std::map<std::pair<int, void *>, at::Tensor>       g_workspaces; // (device, stream) -> float32 tensor, grown on demand

at::Tensor workspace_for(const at::Device &dev, void *stream, int64_t floats)
{
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

} // namespace

PYBIND11_MODULE(_fp6mi_torch, m)
{
    m.doc() = "torch tensors -> fp6mi C ABI";
    m.def("linear_forward_native", &linear_forward_native, pybind11::arg("EXPONENT"), pybind11::arg("MANTISSA"), pybind11::arg("in_feats"),
          pybind11::arg("native_weight"), pybind11::arg("scales"), pybind11::arg("OC"), pybind11::arg("splitK") = 1, pybind11::arg("out") = pybind11::none(),
          pybind11::arg("workspace") = pybind11::none(), pybind11::arg("group_exps") = pybind11::none());
    m.def("clear_workspaces", &clear_workspaces);
}
