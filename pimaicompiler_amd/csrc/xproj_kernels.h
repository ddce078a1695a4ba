// Input projection of one LSTM layer over all time steps, on the gfx950 matrix cores:
//   out[T, N] (fp32) = x[T, K] (fp16) . w[N, K]^T (fp16) + bias[N] (fp32)
// with N = 4H gate rows and K the layer's input width.  Both operands are contiguous along K, which is
// the natural operand layout of v_mfma_f32_16x16x32_f16: lane l of a wavefront supplies 8 consecutive K
// values of row (l % 16), starting at K offset 8 * (l / 16), for A (x) and for B (w) alike, and
// receives out rows 4 * (l / 16) .. + 3 of column (l % 16).
//
// Grid: one block per NT * 16 output columns; its four wavefronts take the 16-row time tiles round-robin
// (MT tiles each), so x is read from cache by every block while w is read from memory once.
// gridDim.y covers T in chunks of 64 * MT steps.  Requirements checked by the launcher: K % 8 == 0,
// 16-byte aligned x and w.
#pragma once

#include "device_common.h"

namespace pimhip
{
template <int MT, int NT>
__global__ __launch_bounds__(256) void input_projection_f16_kernel(const half_t* __restrict__ x,
                                                                  const half_t* __restrict__ w,
                                                                  const float* __restrict__ bias,
                                                                  float* __restrict__ out, int T, int K, int N)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int kq = lane >> 4;  // which 8-wide K slice of a 32-wide step this lane feeds
    const int n_base = blockIdx.x * (NT * 16);
    const int t_base = blockIdx.y * (64 * MT);  // gridDim.y chunks of 64 * MT time steps

    float4_t acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const half_t* xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        int t = t_base + (wave + 4 * m) * 16 + r16;
        if (t > T - 1) t = T - 1;  // rows past T duplicate the last row; they are not stored
        xrow[m] = x + (long)t * K;
    }
    const half_t* wrow[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        int col = n_base + n * 16 + r16;
        if (col > N - 1) col = N - 1;
        wrow[n] = w + (long)col * K;
    }

    half8_t zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;

    for (int k0 = 0; k0 < K; k0 += 32) {
        const int k = k0 + kq * 8;
        const bool k_ok = k < K;  // K % 8 == 0: a lane's 8-wide slice is entirely in or out of range
        half8_t a[MT], b[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) b[n] = k_ok ? *reinterpret_cast<const half8_t*>(wrow[n] + k) : zero;
#pragma unroll
        for (int m = 0; m < MT; ++m) a[m] = k_ok ? *reinterpret_cast<const half8_t*>(xrow[m] + k) : zero;
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m], b[n], acc[m][n], 0, 0, 0);
    }

#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const int col = n_base + n * 16 + r16;
        if (col >= N) continue;
        const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t_base + (wave + 4 * m) * 16 + kq * 4 + i;
                if (t < T) out[(long)t * N + col] = acc[m][n][i] + bv;
            }
        }
    }
}

// bsum[i] = b_ih[i] + b_hh[i] in fp32 (either may be null, meaning zero).
__global__ void lstm_bias_sum_kernel(const half_t* __restrict__ b_ih, const half_t* __restrict__ b_hh,
                                     float* __restrict__ bsum, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) bsum[i] = (b_ih ? (float)b_ih[i] : 0.0f) + (b_hh ? (float)b_hh[i] : 0.0f);
}

}  // namespace pimhip
