// Python access to the C++ operator bodies of aten_ops_pimhip.cpp, so that the GPU tests can drive the exact code a
// maintainer of the reference would link.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <chrono>

#include "../../include/pimhip.h"
#include "aten_ops_pimhip.h"
#include "custom_ops_pimhip.h"

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
    // `iters` calls in a row from C++: what one call costs the host thread (wall time of the loop / iters, in us).  Nothing
    // synchronises inside the loop, so the figure is the host's, not the GPU's.
    //   "addmm": t = {self, mat1, mat2}    "matmul": t = {self, other}    "linear": t = {input, weight[, bias]}
    //   "lstm1": t = {input, h0, c0}, params in LibTorch order with biases, unidirectional, num_layers = params / 4
    //   "lstm1_into": the same through atenLstm1Into with t = {input, h0, c0, output, hy, cy}
    //   "c_abi_gemv": pimhip_execute_gemv itself (the call under the three GEMV operators) with t = {y[N], x[K], w[N, K], b[N]}:
    //   what of an operator's host time is the library's launch and what the operator layer adds on top
    m.def("opHostMicroseconds", [](const std::string& op, std::vector<at::Tensor> t, std::vector<at::Tensor> params, int iters) {
        torch::jit::IValue out;
        std::vector<at::Tensor> hx;
        if (op == "lstm1" || op == "lstm1_into") hx = {t.at(1), t.at(2)};
        const int64_t layers = (int64_t)params.size() / 4;
        const c10::optional<at::Tensor> bias = (op == "linear" && t.size() > 2) ? c10::optional<at::Tensor>(t[2]) : c10::nullopt;
        void* c_abi_stream = op == "c_abi_gemv" ? (void*)c10::hip::getCurrentHIPStream().stream() : nullptr;
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < iters; ++i) {
            if (op == "addmm")
                ops::customAtenAddmm("none", t.at(0), t.at(1), t.at(2), 1, 1, out, nullptr);
            else if (op == "matmul")
                ops::customAtenMatmul(t.at(0), t.at(1), out, nullptr);
            else if (op == "linear")
                ops::atenLinear(t.at(0), t.at(1), bias);
            else if (op == "lstm1")
                ops::atenLstm1(t.at(0), hx, params, true, layers, 0.0, false, false, false);
            else if (op == "lstm1_into")
                ops::atenLstm1Into(t.at(0), hx, params, true, layers, 0.0, false, false, false, t.at(3), t.at(4), t.at(5));
            else if (op == "c_abi_gemv") {
                if (pimhip_execute_gemv(t.at(0).data_ptr(), t.at(1).data_ptr(), t.at(2).data_ptr(), t.at(3).data_ptr(), t.at(2).size(1),
                                        t.at(2).size(0), 0, PIMHIP_ACT_NONE, PIMHIP_W_X_I, c_abi_stream) != PIMHIP_OK)
                    throw utils::NNRuntimeException(pimhip_last_error());
            }
            else
                throw utils::NNRuntimeException("unknown operator " + op);
        }
        const auto t1 = std::chrono::steady_clock::now();
        return std::chrono::duration<double, std::micro>(t1 - t0).count() / (iters > 0 ? iters : 1);
    });
    m.def("atenLstm1Into", [](const at::Tensor& input, std::vector<at::Tensor> hx, std::vector<at::Tensor> params, bool has_biases,
                              int64_t num_layers, double dropout, bool train, bool bidirectional, bool batch_first,
                              c10::optional<at::Tensor> output, c10::optional<at::Tensor> hy, c10::optional<at::Tensor> cy) {
        at::Tensor y = output.value_or(at::Tensor()), hn = hy.value_or(at::Tensor()), cn = cy.value_or(at::Tensor());
        ops::atenLstm1Into(input, hx, params, has_biases, num_layers, dropout, train, bidirectional, batch_first, y, hn, cn);
        return std::make_tuple(y, hn, cn);
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
    // The launchers with the signatures of the reference's custom_ops.h, called as its own code calls them: raw pointers to 16-bit
    // floating-point elements (the reference's are _Float16*, which this host compiler does not have; at::Half has the same
    // bits), sizes, alpha / beta; `stream` 0 is the null stream, as the reference passes it.
    auto f16 = [](const at::Tensor& t) { return static_cast<at::Half*>(t.data_ptr()); };
    auto hs = [](uintptr_t stream) { return reinterpret_cast<hipStream_t>(stream); };
    m.def("rocblas_gemv_template_xAy", [f16, hs](uintptr_t stream, at::Tensor x, at::Tensor A, at::Tensor y, int mm, int n, int k, float alpha, float beta) {
        ops::rocblas_gemv_template_xAy(hs(stream), (const at::Half*)f16(x), (const at::Half*)f16(A), f16(y), mm, n, k, alpha, beta);
    });
    m.def("rocblas_gemv_template_Axy", [f16, hs](uintptr_t stream, at::Tensor A, at::Tensor x, at::Tensor y, int mm, int n, int k, float alpha, float beta) {
        ops::rocblas_gemv_template_Axy(hs(stream), (const at::Half*)f16(A), (const at::Half*)f16(x), f16(y), mm, n, k, alpha, beta);
    });
    m.def("rocblas_addmv_template_xAy", [f16, hs](uintptr_t stream, at::Tensor b, at::Tensor x, at::Tensor A, at::Tensor y, int mm, int n, int k,
                                                   float alpha, float beta, bool relu) {
        ops::rocblas_addmv_template_xAy(hs(stream), (const at::Half*)f16(b), (const at::Half*)f16(x), (const at::Half*)f16(A), f16(y), mm, n, k, alpha,
                                        beta, relu);
    });
    m.def("rocblas_addmv_template_Axy", [f16, hs](uintptr_t stream, at::Tensor b, at::Tensor A, at::Tensor x, at::Tensor y, int mm, int n, int k,
                                                   float alpha, float beta, bool relu) {
        ops::rocblas_addmv_template_Axy(hs(stream), (const at::Half*)f16(b), (const at::Half*)f16(A), (const at::Half*)f16(x), f16(y), mm, n, k, alpha,
                                        beta, relu);
    });
    m.def("custom_add", [f16, hs](uintptr_t stream, at::Tensor A, at::Tensor B, at::Tensor C, int mm, int n, float alpha, bool sym) {
        ops::custom_add(hs(stream), f16(A), f16(B), f16(C), mm, n, alpha, sym, 1, 1, 1, 1);
    });
    m.def("rocblas_bmm_template_xAy", [f16, hs](uintptr_t stream, at::Tensor x, at::Tensor A, at::Tensor y, int mm, int n, int k) {
        ops::rocblas_bmm_template_xAy(hs(stream), (const at::Half*)f16(x), (const at::Half*)f16(A), f16(y), mm, n, k);
    });
    py::register_exception<utils::NNRuntimeException>(m, "NNRuntimeException");
}
