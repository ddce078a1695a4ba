// Input projection of one LSTM layer over all time steps, on the gfx950 matrix cores:
//   out[T, N] (fp32) = x[T, K] (fp16) . w[N, K]^T (fp16) + bias[N] (fp32)
// with N = 4H gate rows and K the layer's input width.  Both operands are contiguous along K, which is
// the natural operand layout of v_mfma_f32_16x16x32_f16: lane l of a wavefront supplies 8 consecutive K
// values of row (l % 16), starting at K offset 8 * (l / 16), for A (x) and for B (w) alike, and
// receives out rows 4 * (l / 16) .. + 3 of column (l % 16).
//
// Grid: one block of 256 lanes per 16 * NT output columns and 64 time steps.  Requirements checked by the launcher:
// K % 8 == 0, 16-byte aligned x and w, row pitches % 8 == 0.
#pragma once

#include "device_common.h"

namespace pimhip
{
// What bounds this kernel is the rate at which one CU can pull bytes in from L2 with fragment-shaped loads (measured:
// about 32 GB/s per CU on MI355X, whatever the loop structure, unrolling or LDS staging), not the matrix cores.  The run
// time is therefore (bytes a block reads) / 32 GB/s, and the tiling minimises that at full CU coverage: a block computes
// 64 time steps x 16 * NT columns and each of its four wavefronts takes a quarter of the K range for the whole tile
// (4 x NT MFMA tiles), i.e. (64 + 16 * NT) x K halves per block (256 KB at K = 1024, NT = 4, against 448 KB for a
// 208 x 16 tile); the four K quarters are added through LDS in a fixed order at the end.
static constexpr int kXprojTile = 64;    // time steps and output columns per block
static constexpr int kXprojKSplit = 4;   // K quarters per block, one per wavefront
static constexpr int kXprojUnroll = 2;   // K steps (of 32) whose 16 fragment loads are issued together

template <int NT>  // column tiles of 16 per block: 4 for long sequences, fewer when there are too few row blocks to fill the CUs
__global__ __launch_bounds__(256) void input_projection_f16_kernel(const half_t* __restrict__ x,
                                                                  const half_t* __restrict__ w,
                                                                  const float* __restrict__ bias,
                                                                  float* __restrict__ out, int T, int K, int N, long ldx,
                                                                  long ldw)
{
    __shared__ __align__(16) float red[kXprojKSplit][4 * NT][64][4];  // [K quarter][4 x NT MFMA tile][lane][4 rows]: up to 64 KB

    const int lane = threadIdx.x & 63;
    const int ks = threadIdx.x >> 6;  // this wavefront's K quarter
    const int r16 = lane & 15;
    const int kq = lane >> 4;  // which 8-wide K slice of a 32-wide MFMA step this lane feeds
    const int n_base = blockIdx.x * (16 * NT);
    const int t_base = blockIdx.y * kXprojTile;

    const half_t* xrow[4];
    const half_t* wrow[NT];
#pragma unroll
    for (int m = 0; m < 4; ++m) xrow[m] = x + (long)min(t_base + m * 16 + r16, T - 1) * ldx;  // rows past T duplicate the last row; not stored
#pragma unroll
    for (int n = 0; n < NT; ++n) wrow[n] = w + (long)min(n_base + n * 16 + r16, N - 1) * ldw;

    half8_t zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;
    float4_t acc[4][NT];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // This wavefront's K range, in steps of 32: [step_begin, step_end).
    const int steps = (K + 31) >> 5;
    const int per_quarter = (steps + kXprojKSplit - 1) / kXprojKSplit;
    const int step_begin = ks * per_quarter;
    const int step_end = min(steps, step_begin + per_quarter);

    for (int s0 = step_begin; s0 < step_end; s0 += kXprojUnroll) {
        half8_t a[kXprojUnroll][4], b[kXprojUnroll][NT];
#pragma unroll
        for (int u = 0; u < kXprojUnroll; ++u) {
            // Within the 32 * kXprojUnroll K values of an iteration lane group kq owns a contiguous run and feeds its
            // u-th 8-wide piece to the u-th K step (x and w alike, so products still pair equal K indices): the four
            // lane groups of a row then cover a whole 128-byte line with back-to-back loads instead of half of it.
            const int k = s0 * 32 + kq * (8 * kXprojUnroll) + u * 8;
            const bool ok = k < step_end * 32 && k < K;  // K % 8 == 0: an 8-wide slice is entirely in or out of range
            const int kc = ok ? k : 0;                     // unconditional loads from a valid address, zeroed when out
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const half8_t av = *reinterpret_cast<const half8_t*>(xrow[m] + kc);
                a[u][m] = ok ? av : zero;
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const half8_t bv = *reinterpret_cast<const half8_t*>(wrow[n] + kc);
                b[u][n] = ok ? bv : zero;
            }
        }
#pragma unroll
        for (int u = 0; u < kXprojUnroll; ++u)
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][m], b[u][n], acc[m][n], 0, 0, 0);
    }

#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) *reinterpret_cast<float4_t*>(&red[ks][m * NT + n][lane][0]) = acc[m][n];
    __syncthreads();

    // Wavefront `ks` now finishes the row tile m = ks: lane (r16, kq) holds rows 4 * kq .. + 3 of column r16 of a tile.
    const int m = ks;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        float4_t v = *reinterpret_cast<const float4_t*>(&red[0][m * NT + n][lane][0]);
#pragma unroll
        for (int q = 1; q < kXprojKSplit; ++q) {
            const float4_t p = *reinterpret_cast<const float4_t*>(&red[q][m * NT + n][lane][0]);
            v[0] += p[0];
            v[1] += p[1];
            v[2] += p[2];
            v[3] += p[3];
        }
        const int col = n_base + n * 16 + r16;
        if (col < N) {
            const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t_base + m * 16 + kq * 4 + i;
                if (t < T) out[(long)t * N + col] = v[i] + bv;
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
