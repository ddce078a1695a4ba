// Test infrastructure.  Compiled twice, once with CUSTOM_OPS_HEADER naming the reference's
// runtime/include/executor/op_executor/custom_ops.h where it lies and once naming pimaicompiler_amd/cpp/custom_ops_pimhip.h:
// the calls below are those the reference's own code makes of these launchers (runtime/unit-tests/custom_op_ut.cpp:42, :64;
// aten_ops_executor.cpp:159, :735; the addmv launchers with the argument lists of custom_ops.h:281-283, 364-366), with its
// argument types.  A launcher whose name, namespace, template parameters or argument order has drifted from the reference's
// fails to compile against one of the two headers.
#include <hip/hip_runtime.h>

#include CUSTOM_OPS_HEADER

using namespace nn_compiler::runtime::op_executor;

void calls_as_the_reference_makes_them(_Float16* x, _Float16* A, _Float16* y, _Float16* b, int m, int n, int k)
{
    float alpha = 1.0f;
    float beta = 0.0f;
    rocblas_gemv_template_xAy(nullptr, x, A, y, m, n, k, alpha, beta);
    rocblas_gemv_template_Axy(nullptr, A, x, y, m, n, k, alpha, beta);
    rocblas_addmv_template_xAy(nullptr, b, x, A, y, m, n, k, alpha, beta, true);
    rocblas_addmv_template_Axy(nullptr, b, A, x, y, m, n, k, alpha, beta, false);
    _Float16* C = y;
    bool sym = true;
    int a_m_s = 1, a_n_s = 1, b_m_s = 1, b_n_s = 1;
    custom_add(nullptr, A, x, C, m, n, alpha, sym, a_m_s, a_n_s, b_m_s, b_n_s);
    rocblas_bmm_template_xAy(nullptr, x, A, y, m, n, k);
    // explicit instantiations with the reference's template parameter lists
    void (*p1)(hipStream_t, const _Float16*, const _Float16*, _Float16*, int, int, int, float, float) = &rocblas_gemv_template_xAy<float, _Float16, _Float16>;
    void (*p2)(hipStream_t, const _Float16*, const _Float16*, _Float16*, int, int, int, float, float) = &rocblas_gemv_template_Axy<float, _Float16, _Float16>;
    void (*p3)(hipStream_t, const _Float16*, const _Float16*, const _Float16*, _Float16*, int, int, int, float, float, bool) =
        &rocblas_addmv_template_xAy<float, _Float16, _Float16>;
    void (*p4)(hipStream_t, const _Float16*, const _Float16*, const _Float16*, _Float16*, int, int, int, float, float, bool) =
        &rocblas_addmv_template_Axy<float, _Float16, _Float16>;
    void (*p5)(hipStream_t, _Float16*, _Float16*, _Float16*, int, int, float, bool, int, int, int, int) = &custom_add<_Float16, float>;
    void (*p6)(hipStream_t, const _Float16*, const _Float16*, _Float16*, int, int, int) = &rocblas_bmm_template_xAy<_Float16, _Float16>;
#ifdef SIGCHECK_DRIFT
    // the control: an argument list neither header declares (the bias after the operands) has to fail against both
    void (*drift)(hipStream_t, const _Float16*, const _Float16*, _Float16*, const _Float16*, int, int, int, float, float, bool) =
        &rocblas_addmv_template_xAy<float, _Float16, _Float16>;
    (void)drift;
#endif
    (void)p1; (void)p2; (void)p3; (void)p4; (void)p5; (void)p6;
}
