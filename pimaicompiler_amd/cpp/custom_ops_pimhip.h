// The launchers of the reference's runtime/include/executor/op_executor/custom_ops.h with their own names, namespace,
// template parameters and argument order, written against the C ABI of include/pimhip.h: with this header in that one's
// place, executeAtenAdd (aten_ops_executor.cpp:159), executeAtenBmm (aten_ops_executor.cpp:735) and the GEMV unit test
// (runtime/unit-tests/custom_op_ut.cpp:42, :64) compile as they are.
//
//   rocblas_gemv_template_xAy   custom_ops.h:123-139    y[1, n] = alpha * x[1, k] . A[k, n] + beta * y
//   rocblas_gemv_template_Axy   custom_ops.h:198-214    y[m, 1] = alpha * A[m, k] . x[k, 1] + beta * y
//   rocblas_addmv_template_xAy  custom_ops.h:281-298    y = relu?(alpha * x . A + beta * y + b)
//   rocblas_addmv_template_Axy  custom_ops.h:364-381    y = relu?(alpha * A . x + beta * y + b)
//   custom_add                  custom_ops.h:415-433    C[m, n] = A[m, n] + B  (B [m, n] when sym, one row [n] otherwise)
//   rocblas_bmm_template_xAy    custom_ops.h:450-466    y[1, n] = x[1, k] . A[k, n]
//
// As in the reference: 16-bit floating-point elements (it passes _Float16*), a null stream is the device's default stream,
// and a call whose m (n for Axy) is not 1 is a matrix-matrix product and does nothing.  Unlike the reference, a failure is
// not silent: it throws std::runtime_error with the library's message.  custom_add ignores alpha and the four strides,
// which the reference's kernels never read either.
#pragma once

#include <hip/hip_runtime_api.h>

#include <stdexcept>
#include <string>

#include "../../include/pimhip.h"

namespace nn_compiler
{
namespace runtime
{
namespace op_executor
{
namespace pimhip_detail
{
inline void check(int rc, const char* what)
{
    if (rc != PIMHIP_OK) throw std::runtime_error(std::string(what) + ": " + pimhip_last_error());
}
template <typename V>
constexpr void half_only()
{
    static_assert(sizeof(V) == 2, "these launchers take 16-bit floating-point elements, as the reference's do");
}
}  // namespace pimhip_detail

template <typename U, typename V, typename W>
void rocblas_gemv_template_xAy(hipStream_t p_stream, const V* x, const V* A, W* y, int m, int n, int k, U alpha, U beta)
{
    pimhip_detail::half_only<V>();
    pimhip_detail::half_only<W>();
    if (m != 1) return;  // found gemm, unsupported
    pimhip_detail::check(pimhip_execute_gemv_scaled(y, x, A, nullptr, k, n, 0, PIMHIP_ACT_NONE, PIMHIP_I_X_W, (float)alpha, (float)beta, p_stream),
                         "rocblas_gemv_template_xAy");
}

template <typename U, typename V, typename W>
void rocblas_gemv_template_Axy(hipStream_t p_stream, const V* A, const V* x, W* y, int m, int n, int k, U alpha, U beta)
{
    pimhip_detail::half_only<V>();
    pimhip_detail::half_only<W>();
    if (n != 1) return;  // found gemm, unsupported
    pimhip_detail::check(pimhip_execute_gemv_scaled(y, x, A, nullptr, k, m, 0, PIMHIP_ACT_NONE, PIMHIP_W_X_I, (float)alpha, (float)beta, p_stream),
                         "rocblas_gemv_template_Axy");
}

template <typename U, typename V, typename W>
void rocblas_addmv_template_xAy(hipStream_t p_stream, const V* b, const V* x, const V* A, W* y, int m, int n, int k, U alpha, U beta,
                                bool relu)
{
    pimhip_detail::half_only<V>();
    pimhip_detail::half_only<W>();
    if (m != 1) return;  // found gemm, unsupported
    pimhip_detail::check(pimhip_execute_gemv_scaled(y, x, A, b, k, n, 0, relu ? PIMHIP_ACT_RELU : PIMHIP_ACT_NONE, PIMHIP_I_X_W, (float)alpha,
                                                    (float)beta, p_stream),
                         "rocblas_addmv_template_xAy");
}

template <typename U, typename V, typename W>
void rocblas_addmv_template_Axy(hipStream_t p_stream, const V* b, const V* A, const V* x, W* y, int m, int n, int k, U alpha, U beta,
                                bool relu)
{
    pimhip_detail::half_only<V>();
    pimhip_detail::half_only<W>();
    if (n != 1) return;  // found gemm, unsupported
    pimhip_detail::check(pimhip_execute_gemv_scaled(y, x, A, b, k, m, 0, relu ? PIMHIP_ACT_RELU : PIMHIP_ACT_NONE, PIMHIP_W_X_I, (float)alpha,
                                                    (float)beta, p_stream),
                         "rocblas_addmv_template_Axy");
}

template <typename U, typename W>
void custom_add(hipStream_t p_stream, U* A, U* B, U* C, int m, int n, W /*alpha*/, bool sym, int /*a_m_s*/, int /*a_n_s*/, int /*b_m_s*/,
                int /*b_n_s*/)
{
    pimhip_detail::half_only<U>();
    pimhip_detail::check(pimhip_execute_add(C, A, B, m, n, sym ? 0 : 1, p_stream), "custom_add");
}

template <typename V, typename W>
void rocblas_bmm_template_xAy(hipStream_t p_stream, const V* x, const V* A, W* y, int m, int n, int k)
{
    pimhip_detail::half_only<V>();
    pimhip_detail::half_only<W>();
    if (m != 1) return;  // found gemm, unsupported
    void* outs[1] = {y};
    pimhip_detail::check(pimhip_execute_bmm(outs, 1, x, A, k, n, p_stream), "rocblas_bmm_template_xAy");
}

}  // namespace op_executor
}  // namespace runtime
}  // namespace nn_compiler
