// TEST INFRASTRUCTURE.  A C-ABI driver around the reference's own HIP GEMV / add / bmm launchers, compiled
// from the reference header where it lies (-I<reference>/ -I<reference>/runtime/include) into
// oracle/_ref/libref_custom_ops.so.  The header is the reference's
// runtime/include/executor/op_executor/custom_ops.h (launchers at :123-139, :198-214, :281-298, :364-381,
// :415-433, :450-466); nothing of it is copied into this repository.  Used by the GPU tests as a second
// checker and by bench.py to time the reference's kernels beside this repository's.
#include "executor/op_executor/custom_ops.h"

using namespace nn_compiler::runtime::op_executor;

extern "C" {

// y[1,n] = x[1,k] . A[k,n]
void ref_gemv_xAy(void* stream, const void* x, const void* A, void* y, int n, int k)
{
    rocblas_gemv_template_xAy((hipStream_t)stream, (const _Float16*)x, (const _Float16*)A, (_Float16*)y, 1, n, k, 1.0f, 0.0f);
}

// y[m,1] = A[m,k] . x[k,1]
void ref_gemv_Axy(void* stream, const void* A, const void* x, void* y, int m, int k)
{
    rocblas_gemv_template_Axy((hipStream_t)stream, (const _Float16*)A, (const _Float16*)x, (_Float16*)y, m, 1, k, 1.0f, 0.0f);
}

// y[1,n] = x . A + b, optional ReLU
void ref_addmv_xAy(void* stream, const void* b, const void* x, const void* A, void* y, int n, int k, int relu)
{
    rocblas_addmv_template_xAy((hipStream_t)stream, (const _Float16*)b, (const _Float16*)x, (const _Float16*)A, (_Float16*)y, 1, n, k, 1.0f, 0.0f, relu != 0);
}

// y[m,1] = A . x + b, optional ReLU
void ref_addmv_Axy(void* stream, const void* b, const void* A, const void* x, void* y, int m, int k, int relu)
{
    rocblas_addmv_template_Axy((hipStream_t)stream, (const _Float16*)b, (const _Float16*)A, (const _Float16*)x, (_Float16*)y, m, 1, k, 1.0f, 0.0f, relu != 0);
}

// C[m,n] = A[m,n] + B ([m,n] if sym else [n] broadcast over rows)
void ref_custom_add(void* stream, void* A, void* B, void* C, int m, int n, int sym)
{
    custom_add((hipStream_t)stream, (_Float16*)A, (_Float16*)B, (_Float16*)C, m, n, 1.0f, sym != 0, 0, 0, 0, 0);
}

// y[1,n] = x[1,k] . A[k,n] (fp16 accumulator)
void ref_bmm_xAy(void* stream, const void* x, const void* A, void* y, int n, int k)
{
    rocblas_bmm_template_xAy((hipStream_t)stream, (const _Float16*)x, (const _Float16*)A, (_Float16*)y, 1, n, k);
}

}  // extern "C"
