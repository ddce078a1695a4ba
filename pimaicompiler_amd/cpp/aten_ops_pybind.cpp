// Python access to the C++ operator bodies of aten_ops_pimhip.cpp, so that the GPU tests can drive the exact code a
// maintainer of the reference would link.
#include <torch/extension.h>

#include <chrono>

#include "aten_ops_pimhip.h"

namespace ops = nn_compiler::runtime::op_executor;
namespace utils = nn_compiler::runtime::utils;

PYBIND11_MODULE(_aten_ops_pimhip, m)
{
    m.def("initialize", &ops::pimhipRuntimeInitialize);
    m.def("deinitialize", &ops::pimhipRuntimeDeinitialize);
    m.def("invalidateLstmPlans", [](std::vector<at::Tensor> params) { return ops::pimhipInvalidateLstmPlans(params); });
    m.def("customAtenAddmm", [](const std::string& act, at::Tensor self, at::Tensor mat1, at::Tensor mat2, double beta, double alpha) {
        torch::jit::IValue out;
        ops::customAtenAddmm(act, self, mat1, mat2, beta, alpha, out, nullptr);
        return out.toTensor();
    });
    // `iters` calls in a row from C++: what one call costs the host thread (wall time of the loop / iters, in us).
    m.def("customAtenAddmmHostMicroseconds", [](const std::string& act, at::Tensor self, at::Tensor mat1, at::Tensor mat2, int iters) {
        torch::jit::IValue out;
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < iters; ++i) ops::customAtenAddmm(act, self, mat1, mat2, 1, 1, out, nullptr);
        const auto t1 = std::chrono::steady_clock::now();
        return std::chrono::duration<double, std::micro>(t1 - t0).count() / (iters > 0 ? iters : 1);
    });
    m.def("customAtenMatmul", [](at::Tensor self, at::Tensor other) {
        torch::jit::IValue out;
        ops::customAtenMatmul(self, other, out, nullptr);
        return out.toTensor();
    });
    m.def("atenLinear", [](const at::Tensor& x, const at::Tensor& w, const c10::optional<at::Tensor>& b) {
        return ops::atenLinear(x, w, b);
    });
    m.def("atenLstm1", [](const at::Tensor& input, std::vector<at::Tensor> hx, std::vector<at::Tensor> params, bool has_biases,
                          int64_t num_layers, double dropout, bool train, bool bidirectional, bool batch_first) {
        return ops::atenLstm1(input, hx, params, has_biases, num_layers, dropout, train, bidirectional, batch_first);
    });
    m.def("atenLstm2", [](const at::Tensor& data, const at::Tensor& batch_sizes, std::vector<at::Tensor> hx,
                          std::vector<at::Tensor> params, bool has_biases, int64_t num_layers, double dropout, bool train,
                          bool bidirectional) {
        return ops::atenLstm2(data, batch_sizes, hx, params, has_biases, num_layers, dropout, train, bidirectional);
    });
    m.def("gemmBroadcast", [](std::vector<int64_t> a, std::vector<int64_t> b) {
        utils::gemmBroadcast(a, b);
        return std::make_pair(a, b);
    });
    m.def("getGemmType", [](std::vector<int64_t> a, std::vector<int64_t> b) { return (int)utils::getGemmType(a, b); });
    py::register_exception<utils::NNRuntimeException>(m, "NNRuntimeException");
}
