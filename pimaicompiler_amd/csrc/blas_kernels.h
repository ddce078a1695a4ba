// y = act(alpha * (weight . x) + beta * y + bias) for any alpha and beta (gfx950, fp16 storage, fp32 sums, one rounding at
// the store): the general form of the launchers in the reference's runtime/include/executor/op_executor/custom_ops.h
// (gemvt_kernel_calc_xAy / _Axy :66-108, :142-183; addmv_kernel_calc_* :216-259, :300-342).  The reference itself only ever
// passes alpha = 1, beta = 0, which the GEMV kernels of gemv_kernels.h serve; these two kernels exist so that the other
// values are served too.  They are plain: one wavefront per output row (MV order), one lane per output column (VM order),
// 2-byte loads, no requirement on sizes, pitch or alignment.
#pragma once

#include "device_common.h"

namespace pimhip
{

// MV order: weight [N, K] with row pitch ldw; one wavefront per row.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_mv_scaled_f16_kernel(const half_t* __restrict__ W, const half_t* __restrict__ x,
                                                                        const half_t* __restrict__ bias, half_t* y, int N, int K,
                                                                        long ldw, int relu, float alpha, float beta)
{
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * WAVES + (threadIdx.x >> 6);
    if (row >= N) return;
    const half_t* w = W + row * ldw;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) acc = fmaf((float)w[k], (float)x[k], acc);
    acc = wave_sum(acc);
    if (lane == 0) {
        float v = alpha * acc;
        if (beta != 0.0f) v += beta * (float)y[row];  // (as the reference: y is not read when beta is 0)
        if (bias) v += (float)bias[row];
        if (relu) v = relu_f32(v);
        y[row] = (half_t)v;
    }
}

// VM order: weight [K, N] with row pitch lda; a block of 16 wavefronts owns 64 adjacent output columns (one per lane),
// wavefront g takes the rows g, g + 16, ... and the sixteen partial sums meet in LDS.
static constexpr int kVmScaledWaves = 16;
__global__ __launch_bounds__(64 * kVmScaledWaves) void gemv_vm_scaled_f16_kernel(const half_t* __restrict__ x, const half_t* __restrict__ A,
                                                                                 const half_t* __restrict__ bias, half_t* y, int K, int N,
                                                                                 long lda, int relu, float alpha, float beta)
{
    __shared__ float red[kVmScaledWaves][64];
    const int lane = threadIdx.x & 63;
    const int g = threadIdx.x >> 6;
    const long col = (long)blockIdx.x * 64 + lane;
    float acc = 0.0f;
    if (col < N)
        for (int k = g; k < K; k += kVmScaledWaves) acc = fmaf((float)A[(long)k * lda + col], (float)x[k], acc);
    red[g][lane] = acc;
    __syncthreads();
    if (g == 0 && col < N) {
        float s = red[0][lane];
#pragma unroll
        for (int w = 1; w < kVmScaledWaves; ++w) s += red[w][lane];
        float v = alpha * s;
        if (beta != 0.0f) v += beta * (float)y[col];
        if (bias) v += (float)bias[col];
        if (relu) v = relu_f32(v);
        y[col] = (half_t)v;
    }
}

}  // namespace pimhip
