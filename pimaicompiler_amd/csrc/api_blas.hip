// The GEMV of the C ABI (include/pimhip.h) with the alpha and beta of the reference's own launchers.
#include "api_common.h"
#include "blas_kernels.h"

using namespace pimhip;

extern "C" int pimhip_execute_gemv_scaled(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                                          int64_t out_w, int64_t ld_weight, int act, int order, float alpha, float beta,
                                          void* stream)
{
    if (alpha == 1.0f && beta == 0.0f) return pimhip_execute_gemv(out, in, weight, bias, in_w, out_w, ld_weight, act, order, stream);
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !in || !weight) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, in and weight must be non-null");
    if (in_w < 0 || out_w < 0 || in_w > INT32_MAX || out_w > INT32_MAX)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in_w=%lld out_w=%lld out of range", (long long)in_w, (long long)out_w);
    if (act != PIMHIP_ACT_NONE && act != PIMHIP_ACT_RELU) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown activation %d", act);
    if (order != PIMHIP_I_X_W && order != PIMHIP_W_X_I) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown operand order %d", order);
    if (out_w == 0) return PIMHIP_OK;
    const int64_t dense = (order == PIMHIP_W_X_I) ? in_w : out_w;
    if (ld_weight == 0) ld_weight = dense;
    if (ld_weight < dense)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ld_weight=%lld is below the row length %lld", (long long)ld_weight, (long long)dense);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int relu = act == PIMHIP_ACT_RELU;
    if (order == PIMHIP_W_X_I)
        gemv_mv_scaled_f16_kernel<4><<<(unsigned)((out_w + 3) / 4), 256, 0, s>>>((const half_t*)weight, (const half_t*)in, (const half_t*)bias,
                                                                                 (half_t*)out, (int)out_w, (int)in_w, (long)ld_weight, relu, alpha, beta);
    else
        gemv_vm_scaled_f16_kernel<<<(unsigned)((out_w + 63) / 64), 64 * kVmScaledWaves, 0, s>>>((const half_t*)in, (const half_t*)weight,
                                                                                               (const half_t*)bias, (half_t*)out, (int)in_w, (int)out_w,
                                                                                               (long)ld_weight, relu, alpha, beta);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}
