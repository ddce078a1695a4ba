// A stack of LSTM layers over a whole sequence computed by ONE workgroup, without any other workgroup's help.
//
// The persistent sequence kernels (lstm_kernels.h, lstm_xcd_kernels.h) split a recurrence over many workgroups that hand
// each other h once per step and therefore have to run at the same time.  When one of their bounded waits gives up (other
// work kept part of the GPU from running them together), the workgroup that waited in vain does not leave its outputs
// undefined: it stops publishing, and at the end of the launch it recomputes the whole stack from the call's inputs here,
// alone, and stores the units it owns.  That is slow (every step streams the layers' weights through one compute unit:
// tens of microseconds per layer-step instead of one) but it needs nobody, so it always ends, and the call's result is
// what it would have been.  Workgroups whose waits all succeeded have consumed only values that were really computed
// (a workgroup that gave up publishes nothing from then on) and keep what they stored.
//
// Arithmetic as in lstm_step_f16_kernel: exact products, fp32 sums, h rounded to fp16 once per step, c in fp32.
#pragma once

#include "device_common.h"

namespace pimhip
{
static constexpr int kSoloMaxLayers = 4;

struct SoloLayer {
    const half_t* w_hh;   // [4H, H]
    const half_t* w_ih;   // [4H, H]; null for the first layer of the stack (its input projection is given)
    const float* bsum;    // [4H] fp32 b_ih + b_hh; with w_ih
    const half_t* h0;     // [H]
    const half_t* c0;     // [H]
    half_t* y;            // row t at y + t * y_stride, or null
    half_t* hn;           // [H]
    half_t* cn;           // [H]
    int residual;         // 1: the layer hands up and stores out_t = h_t + in_t (in_t: its own input); hn stays h
    int u_begin, u_end;   // the units of this layer whose y / hn / cn this workgroup stores (empty range: none)
};

struct SoloStack {
    SoloLayer layer[kSoloMaxLayers];
    int n;                   // layers
    const float* xproj;      // [T, 4H] fp32, biases included: the first layer's input projection, row t
    const half_t* res_in0;   // [T, H]: the first layer's own input, when it has a residual sum
    int reverse;             // 1: steps run over t = T - 1 .. 0
    long y_stride;
    int H, T;
};

// Every thread of the workgroup calls this (THREADS threads, a multiple of 64).  MAXH >= H.
template <int THREADS, int MAXL, int MAXH>
__device__ __forceinline__ void lstm_solo_stack(const SoloStack& desc)
{
    constexpr int WAVES = THREADS / 64;
    // The description is read from LDS (the loops below index its layers with a run-time index).
    __shared__ SoloStack s;
    __syncthreads();
    if (threadIdx.x == 0) s = desc;
    __shared__ __align__(16) half_t solo_h[2][MAXL][MAXH];  // h of every layer, double buffered by step parity
    __shared__ __align__(16) half_t solo_out[MAXL][MAXH];   // what every layer hands up in this step (h, or h + in)
    __shared__ float solo_c[MAXL][MAXH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __syncthreads();
    const int H = s.H, T = s.T, nchunks = H >> 3;
    for (int l = 0; l < s.n; ++l) {
        for (int u = tid; u < MAXH; u += THREADS) {
            solo_h[0][l][u] = u < H ? s.layer[l].h0[u] : (half_t)0.0f;
            solo_h[1][l][u] = (half_t)0.0f;
            solo_out[l][u] = (half_t)0.0f;
            solo_c[l][u] = u < H ? (float)s.layer[l].c0[u] : 0.0f;
        }
    }
    __syncthreads();
    for (int step = 0; step < T; ++step) {
        const int t = s.reverse ? (T - 1 - step) : step;
        const int cur = step & 1, nxt = cur ^ 1;
        for (int l = 0; l < s.n; ++l) {
            const SoloLayer& ly = s.layer[l];
            const half8_t* hv = reinterpret_cast<const half8_t*>(&solo_h[cur][l][0]);
            const half8_t* iv = l > 0 ? reinterpret_cast<const half8_t*>(&solo_out[l - 1][0]) : nullptr;
            for (int u = wave; u < H; u += WAVES) {
                float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                for (int c = lane; c < nchunks; c += 64) {
                    const half8_t h8 = hv[c];
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        acc[g] = dot8(*reinterpret_cast<const half8_t*>(ly.w_hh + ((long)g * H + u) * H + c * 8), h8, acc[g]);
                    if (l > 0) {
                        const half8_t x8 = iv[c];
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            acc[g] = dot8(*reinterpret_cast<const half8_t*>(ly.w_ih + ((long)g * H + u) * H + c * 8), x8, acc[g]);
                    }
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) acc[g] = wave_sum(acc[g]);
                if (lane == 0) {
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        acc[g] += l > 0 ? ly.bsum[(long)g * H + u] : s.xproj[(long)t * 4 * H + (long)g * H + u];
                    const float c_new = sigmoid_f32(acc[1]) * solo_c[l][u] + sigmoid_f32(acc[0]) * tanh_f32(acc[2]);
                    const half_t h_new = (half_t)(sigmoid_f32(acc[3]) * tanh_f32(c_new));
                    solo_c[l][u] = c_new;
                    solo_h[nxt][l][u] = h_new;
                    half_t out = h_new;
                    if (ly.residual) {
                        const half_t in = l > 0 ? solo_out[l - 1][u] : s.res_in0[(long)t * H + u];
                        out = (half_t)((float)h_new + (float)in);
                    }
                    solo_out[l][u] = out;
                    if (u >= ly.u_begin && u < ly.u_end) {
                        if (ly.y) ly.y[(long)t * s.y_stride + u] = out;
                        if (step == T - 1) {
                            ly.hn[u] = h_new;
                            ly.cn[u] = (half_t)c_new;
                        }
                    }
                }
            }
            __syncthreads();  // this layer's output of the step is complete before the next layer reads it
        }
    }
}

}  // namespace pimhip
