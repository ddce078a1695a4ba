// LSTM kernels for gfx950, batch 1, fp16 storage, fp32 gates and cell state.
//
// Cell (gate order i, f, g, o as in LibTorch's at::lstm, which the reference calls from atenLstm1/2,
// runtime/source/executor/op_executor/aten_ops.cpp:328-344):
//   a   = W_ih x_t + b_ih + W_hh h_{t-1} + b_hh          (4H pre-activations)
//   c_t = sigmoid(a_f) * c_{t-1} + sigmoid(a_i) * tanh(a_g)
//   h_t = sigmoid(a_o) * tanh(c_t)
// h_t is rounded to fp16 once per step (it is fp16 at the interface); c stays fp32 inside a sequence.
//
// Two ways to run the recurrence:
//   lstm_step_f16_kernel      one launch per (layer, direction, step): streams W_hh (and W_ih when the
//                             input projection is fused) once, HBM-bound.  Used for seq_len == 1 decode
//                             steps and as the fallback for shapes the persistent kernel does not take.
//   lstm_seq_f16_kernel       one launch per (layer, direction) for the whole sequence: every block keeps
//                             its 16 rows of W_hh in LDS and its cell state in registers for all steps; h_t
//                             is exchanged between blocks through tagged words in device memory, so
//                             the per-step cost is one device-scope store/load round trip, not a launch.
#pragma once

#include "device_common.h"

namespace pimhip
{
// ---------------------------------------------------------------------------------------------
// Single step.  One wavefront per hidden unit j: its four gate rows j, H+j, 2H+j, 3H+j.
//   xproj  != nullptr : a = xproj[4H] (fp32, biases included) + W_hh h
//   xproj  == nullptr : a = W_ih x + W_hh h + bsum[4H] (fp32 or nullptr)
// Requirements checked by the launcher: H % 8 == 0, I % 8 == 0, 16-byte aligned pointers.
// c_in_f16 (fp16) is read when non-null, else c_state (fp32); c_state is always written; h_out, and
// hn_f16 / cn_f16 when non-null, receive the new state.
// ---------------------------------------------------------------------------------------------
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void lstm_step_f16_kernel(
    const half_t* __restrict__ w_ih, const half_t* __restrict__ w_hh, const float* __restrict__ bsum,
    const float* __restrict__ xproj, const half_t* __restrict__ x, const half_t* __restrict__ h_prev,
    const half_t* __restrict__ c_in_f16, float* __restrict__ c_state, half_t* __restrict__ h_out,
    half_t* __restrict__ hn_f16, half_t* __restrict__ cn_f16, int I, int H)
{
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * WAVES + (threadIdx.x >> 6);
    if (j >= H) return;

    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    {
        const half8_t* hv = reinterpret_cast<const half8_t*>(h_prev);
        const half8_t* w0 = reinterpret_cast<const half8_t*>(w_hh + (long)j * H);
        const long gstride = (long)H * H / 8;  // one gate block of rows, in 16-byte units
        const int nchunks = H >> 3;
        int c = lane;
        for (; c + 64 < nchunks; c += 128) {
            half8_t wr[4][2];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                wr[g][0] = load_stream(w0 + g * gstride + c);
                wr[g][1] = load_stream(w0 + g * gstride + c + 64);
            }
            const half8_t h0 = hv[c], h1 = hv[c + 64];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g][1], h1, dot8(wr[g][0], h0, acc[g]));
        }
        for (; c < nchunks; c += 64) {
            half8_t wr[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) wr[g] = load_stream(w0 + g * gstride + c);
            const half8_t h0 = hv[c];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g], h0, acc[g]);
        }
    }
    if (xproj == nullptr) {
        const half8_t* xv = reinterpret_cast<const half8_t*>(x);
        const half8_t* w0 = reinterpret_cast<const half8_t*>(w_ih + (long)j * I);
        const long gstride = (long)H * I / 8;
        const int nchunks = I >> 3;
        int c = lane;
        for (; c + 64 < nchunks; c += 128) {
            half8_t wr[4][2];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                wr[g][0] = load_stream(w0 + g * gstride + c);
                wr[g][1] = load_stream(w0 + g * gstride + c + 64);
            }
            const half8_t x0 = xv[c], x1 = xv[c + 64];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g][1], x1, dot8(wr[g][0], x0, acc[g]));
        }
        for (; c < nchunks; c += 64) {
            half8_t wr[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) wr[g] = load_stream(w0 + g * gstride + c);
            const half8_t x0 = xv[c];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g], x0, acc[g]);
        }
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) acc[g] = wave_sum(acc[g]);

    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (xproj)
                acc[g] += xproj[(long)g * H + j];
            else if (bsum)
                acc[g] += bsum[(long)g * H + j];
        }
        const float c_prev = c_in_f16 ? (float)c_in_f16[j] : c_state[j];
        const float c_new = sigmoid_f32(acc[1]) * c_prev + sigmoid_f32(acc[0]) * tanh_f32(acc[2]);
        const half_t h_new = (half_t)(sigmoid_f32(acc[3]) * tanh_f32(c_new));
        c_state[j] = c_new;
        h_out[j] = h_new;
        if (hn_f16) hn_f16[j] = h_new;
        if (cn_f16) cn_f16[j] = (half_t)c_new;
    }
}

// ---------------------------------------------------------------------------------------------
// Whole sequence, one (layer, direction).
//
// Grid: NB = ceil(H / 4) blocks of 256 lanes (H <= 1024, H % 8 == 0), all resident at once.  Block b owns
// hidden units 4b .. 4b+3, i.e. 16 gate rows of W_hh, held in LDS as `slot = 4 * unit + gate` rows of H
// halves.  Lane t of the block owns columns 4t .. 4t+3 of every row, which are exactly the four h values
// block t produces.
//
// Exchange buffer: hx[2][NB][2] 64-bit words, word = (tag << 32) | two fp16 values.  Step s of a launch
// publishes its h under tag `tag_base + s + 1` into parity s & 1; step s >= 1 waits until both words of
// its entry in parity (s - 1) & 1 carry tag `tag_base + s`.  Data and flag travel in one word, written
// and read with device-scope relaxed atomics (which go to memory past the per-XCD L2), so one store/load
// round trip publishes a step.  A block cannot overwrite parity p before every block has consumed it:
// writing step s + 2 needs h of step s + 1 from all blocks, which they publish only after reading step s.
// The host advances tag_base by seq_len per launch, so tags left by earlier launches never match.
//
// Every wait is bounded: after `spin_limit` polls a lane raises *abort_flag and stops waiting; lanes poll
// the flag every 256 spins and stop waiting once it is set.  The kernel then runs to the end with
// undefined results and the host reports a time-out.
// ---------------------------------------------------------------------------------------------
static constexpr int kSeqUnits = 4;   // hidden units per block
static constexpr int kSeqRows = 16;   // gate rows per block
static constexpr int kSeqMaxH = 1024; // 256 lanes x 4 columns

// Exchange of a register with the lane whose index differs in bit 2 (xor 4) inside a row of 16 lanes.
__device__ __forceinline__ float dpp_xor4_f32(float v)
{
    int iv = __builtin_bit_cast(int, v);
    // row_ror:4 delivers lane i-4 (taken by lanes with bit 2 set: banks 1 and 3),
    // row_ror:12 delivers lane i+4 (taken by lanes with bit 2 clear: banks 0 and 2).
    int r = __builtin_amdgcn_update_dpp(0, iv, 0x124, 0xf, 0xA, false);
    r = __builtin_amdgcn_update_dpp(r, iv, 0x12C, 0xf, 0x5, false);
    return __builtin_bit_cast(float, r);
}

__device__ __forceinline__ float dpp_xor8_f32(float v)
{
    // row_ror:8 is the xor-8 exchange inside a row of 16 lanes.
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
}

__device__ __forceinline__ float dpp_xor1_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kDppQuadXor1, 0xf, 0xf, false));
}

__device__ __forceinline__ float dpp_xor2_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kDppQuadXor2, 0xf, 0xf, false));
}

// Sums 16 per-lane values over each row of 16 lanes so that lane r of the row ends up with the row total of
// value index  8*bit0(r) + 4*bit1(r) + 2*bit3(r) + bit2(r).  15 exchanges instead of 64.
__device__ __forceinline__ float row16_transpose_sum(const float (&v)[16], int lane)
{
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
    float a[8], b[4], c[2];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float keep = b0 ? v[i + 8] : v[i];
        const float give = b0 ? v[i] : v[i + 8];
        a[i] = keep + dpp_xor1_f32(give);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float keep = b1 ? a[i + 4] : a[i];
        const float give = b1 ? a[i] : a[i + 4];
        b[i] = keep + dpp_xor2_f32(give);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float keep = b3 ? b[i + 2] : b[i];
        const float give = b3 ? b[i] : b[i + 2];
        c[i] = keep + dpp_xor8_f32(give);
    }
    const float keep = b2 ? c[1] : c[0];
    const float give = b2 ? c[0] : c[1];
    return keep + dpp_xor4_f32(give);
}

// Value index held by lane r (0..15) of a row after row16_transpose_sum.
__host__ __device__ constexpr int row16_value_index(int r)
{
    return 8 * (r & 1) + 4 * ((r >> 1) & 1) + 2 * ((r >> 3) & 1) + ((r >> 2) & 1);
}

struct LstmSeqArgs {
    const half_t* w_hh;       // [4H, H]
    const float* xproj;       // [T, 4H] fp32, biases included
    const half_t* h0;         // [H]
    const half_t* c0;         // [H]
    half_t* y;                // row t at y + t * y_stride
    half_t* hn;               // [H]
    half_t* cn;               // [H]
    unsigned long long* hx;   // [2][NB][2]
    unsigned int* abort_flag; // set to 1 when a wait gives up
    long y_stride;            // elements between consecutive time steps of y
    int H;
    int T;
    int reverse;              // 1: process t = T-1 .. 0
    unsigned int tag_base;
    unsigned int spin_limit;
};

__global__ __launch_bounds__(256) void lstm_seq_f16_kernel(LstmSeqArgs p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    half_t* wl = reinterpret_cast<half_t*>(smem_raw);                        // [16][H]
    float* red_base = reinterpret_cast<float*>(smem_raw + (size_t)kSeqRows * p.H * sizeof(half_t));  // [2][16 partials][16 slots]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int H = p.H;
    const int nb = gridDim.x;
    const int j0 = blockIdx.x * kSeqUnits;

    // ---- stage this block's 16 rows of W_hh into LDS (zero rows for units past H) ----
    {
        const int chunks_per_row = H >> 3;
        const int total = kSeqRows * chunks_per_row;
        for (int i = tid; i < total; i += 256) {
            const int slot = i / chunks_per_row;
            const int cc = i - slot * chunks_per_row;
            const int unit = slot >> 2, gate = slot & 3;
            half8_t w;
#pragma unroll
            for (int e = 0; e < 8; ++e) w[e] = (half_t)0.0f;
            if (j0 + unit < H) w = *reinterpret_cast<const half8_t*>(p.w_hh + ((long)gate * H + j0 + unit) * H + cc * 8);
            *reinterpret_cast<half8_t*>(wl + (long)slot * H + cc * 8) = w;
        }
    }
    __syncthreads();

    // Column ownership: lane t owns columns 4t..4t+3 <=> the h values of block t.
    const bool has_cols = tid < nb;
    // Final-stage roles (wave 0, lanes 0..15): lane v finishes slot v = 4 * unit + gate.
    const int my_unit = (lane >> 2) & 3;
    const int my_gate = lane & 3;
    const bool unit_ok = (j0 + my_unit) < H;
    float c_reg = 0.0f;
    if (wave == 0 && lane < 16 && unit_ok) c_reg = (float)p.c0[j0 + my_unit];

    bool gave_up = false;
    const int row_in_wave = lane >> 4;                         // which row of 16 lanes
    const int my_value = row16_value_index(lane & 15);         // slot this lane holds after the transpose-sum

    for (int s = 0; s < p.T; ++s) {
        const int t = p.reverse ? (p.T - 1 - s) : s;

        // Prefetch the input-projection term of this step (independent of h).
        float xp = 0.0f;
        if (wave == 0 && lane < 16 && unit_ok) xp = p.xproj[(long)t * 4 * H + (long)my_gate * H + j0 + my_unit];

        // ---- obtain h_{s-1}: this lane's four columns ----
        half4_t hv;
        hv[0] = hv[1] = hv[2] = hv[3] = (half_t)0.0f;
        if (has_cols) {
            if (s == 0) {
                // H % 8 == 0, so a block's four units are either all valid or the entry ends at H.
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (tid * 4 + e < H) hv[e] = p.h0[tid * 4 + e];
            } else {
                const unsigned int want = p.tag_base + (unsigned int)s;
                unsigned long long* src = p.hx + ((long)((s - 1) & 1) * nb + tid) * 2;
                unsigned long long w0 = 0, w1 = 0;
                unsigned int spins = 0;
                while (true) {
                    w0 = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w1 = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (((unsigned int)(w0 >> 32) == want && (unsigned int)(w1 >> 32) == want) || gave_up) break;
                    ++spins;
                    if ((spins & 255u) == 0u) {
                        if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                    }
                    if (spins >= p.spin_limit) {
                        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        gave_up = true;
                    }
                }
                const unsigned int lo0 = (unsigned int)w0, lo1 = (unsigned int)w1;
                const half2_t p0 = __builtin_bit_cast(half2_t, lo0);
                const half2_t p1 = __builtin_bit_cast(half2_t, lo1);
                hv[0] = p0[0];
                hv[1] = p0[1];
                hv[2] = p1[0];
                hv[3] = p1[1];
            }
        }

        // ---- 16 partial dot products over this lane's 4 columns ----
        float part[16];
        {
            const half_t* wrow = wl + tid * 4;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                half4_t w = has_cols ? *reinterpret_cast<const half4_t*>(wrow + (long)v * H) : hv;
                part[v] = dot4(w, hv, 0.0f);
            }
        }

        // ---- reduce over the 256 lanes: transpose-sum inside rows of 16, then LDS across the 16 rows ----
        // `red` is double buffered by step parity: a wavefront that owns no columns does not wait for h and
        // may already be writing step s + 1 while wave 0 still reads step s; the barrier below keeps it from
        // getting further ahead than that.
        float* red = red_base + (s & 1) * 256;
        const float rowsum = row16_transpose_sum(part, lane);
        red[(wave * 4 + row_in_wave) * 16 + my_value] = rowsum;
        __syncthreads();

        if (wave == 0) {
            float a = 0.0f;
            if (lane < 16) {
                float q[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) q[i] = red[i * 16 + lane];
                a = (((q[0] + q[1]) + (q[2] + q[3])) + ((q[4] + q[5]) + (q[6] + q[7]))) +
                    (((q[8] + q[9]) + (q[10] + q[11])) + ((q[12] + q[13]) + (q[14] + q[15])));
                a += xp;
            }
            // Gather the four gates of a unit inside its quad (slot = 4 * unit + gate).
            const int ai = __builtin_bit_cast(int, a);
            const float a_i = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, ai, 0x00, 0xf, 0xf, false));
            const float a_f = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, ai, 0x55, 0xf, 0xf, false));
            const float a_g = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, ai, 0xAA, 0xf, 0xf, false));
            const float a_o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, ai, 0xFF, 0xf, 0xf, false));
            const float c_new = sigmoid_f32(a_f) * c_reg + sigmoid_f32(a_i) * tanh_f32(a_g);
            const half_t h_new = (half_t)(sigmoid_f32(a_o) * tanh_f32(c_new));
            c_reg = c_new;
            // Lanes 4u (gate lane 0 of unit u) now hold h of unit u; fetch the neighbour unit's h for packing.
            const unsigned int hbits = (unsigned int)__builtin_bit_cast(unsigned short, h_new);
            const unsigned int hnext = (unsigned int)__builtin_amdgcn_update_dpp(0, (int)hbits, 0x104, 0xf, 0xf, true);  // row_shl:4 -> lane i+4
            if (lane == 0 || lane == 8) {
                const unsigned long long word =
                    ((unsigned long long)(p.tag_base + (unsigned int)s + 1u) << 32) | (unsigned long long)(hbits | (hnext << 16));
                unsigned long long* dst = p.hx + ((long)(s & 1) * nb + blockIdx.x) * 2 + (lane >> 3);
                __hip_atomic_store(dst, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (lane < 16 && my_gate == 0 && unit_ok) {
                p.y[(long)t * p.y_stride + j0 + my_unit] = h_new;
                if (s == p.T - 1) {
                    p.hn[j0 + my_unit] = h_new;
                    p.cn[j0 + my_unit] = (half_t)c_new;
                }
            }
        }
    }
}

}  // namespace pimhip
