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
// hidden units 4b .. 4b+3, one per wavefront: wavefront w keeps the four gate rows of unit 4b+w in registers
// for the whole sequence (lane l holds columns 16l .. 16l+15 of each row) and its cell state in a register.
//
// A step:
//   1. lane t of the block (t < NB) obtains the four h values of block t from the exchange buffer (below)
//      and puts them into LDS; one barrier; every wavefront reads the whole h from LDS;
//   2. 4 rows x 16 columns of dot products per lane, a transpose-sum over the 64 lanes (7 exchanges) that
//      leaves gate k in lane k, the four activations in parallel in lanes 0..3, the cell update;
//   3. lane 0 of each wavefront publishes its h value and stores y.
//
// Exchange buffer: hx[2][NB][16] 32-bit words; block b uses words 0..3 of its 64-byte entry (one per unit;
// entries of different blocks do not share a 64-byte segment, which measurably shortens the exchange).
// word = fp16 bits | tag << 16.  Step s of a launch publishes under tag (tag_base + s + 1) & 0xffff into
// parity s & 1; step s >= 1 waits until the four words of an entry in parity (s - 1) & 1 carry tag
// (tag_base + s) & 0xffff.  Data and flag travel in one word, written and read with device-scope relaxed
// atomics, so one store / load round trip through memory publishes a step.  A block cannot overwrite parity
// p before every block has consumed it: publishing step s + 2 needs h of step s + 1 from all blocks, which
// they publish only after reading step s.  The host advances tag_base by seq_len per launch (seq_len <=
// 65000), so the tags left behind by earlier launches (at most tag_base) never equal an expected one.
//
// Every wait is bounded: after `spin_limit` polls a lane raises *abort_flag and stops waiting; lanes poll
// the flag every 256 spins and stop waiting once it is set.  The kernel then runs to the end with
// undefined results and the host reports a time-out.
// ---------------------------------------------------------------------------------------------
static constexpr int kSeqUnits = 4;        // hidden units per block, one per wavefront
static constexpr int kSeqMaxH = 1024;      // 64 lanes x 16 columns
static constexpr int kSeqEntryWords = 16;  // 32-bit words between the entries of consecutive blocks (64 bytes)
static constexpr int kSeqMaxT = 65000;

template <int CTRL>
__device__ __forceinline__ float dpp_mov_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Sum over all lanes that share (lane & 3); every lane receives the total of its class.
__device__ __forceinline__ float wave_sum_mod4(float v)
{
    v += dpp_mov_f32<0x124>(v);  // row_ror:4
    v += dpp_mov_f32<0x128>(v);  // row_ror:8  -> total over the four quads of a row of 16 lanes
    // v_permlane16_swap a, b exchanges rows 1 and 3 of a with rows 0 and 2 of b; v_permlane32_swap a, b exchanges the
    // upper 32 lanes of a with the lower 32 lanes of b.  With a == b == v on entry, a + b is the pairwise sum in
    // every lane.  (Written as asm: the compiler's builtin returns the first result twice.)
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = a + b;
    }
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = a + b;
    }
    return v;
}

struct LstmSeqArgs {
    const half_t* w_hh;       // [4H, H]
    const float* xproj;       // [T, 4H] fp32, biases included
    const half_t* h0;         // [H]
    const half_t* c0;         // [H]
    half_t* y;                // row t at y + t * y_stride
    half_t* hn;               // [H]
    half_t* cn;               // [H]
    unsigned int* hx;         // [2][NB][kSeqEntryWords]
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
    __shared__ __align__(16) half_t hbuf[2][kSeqMaxH];  // h of the previous step, double buffered by step parity

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int H = p.H;
    const int nb = gridDim.x;
    const int j = blockIdx.x * kSeqUnits + wave;  // this wavefront's hidden unit
    const bool unit_ok = j < H;

    // ---- this wavefront's four gate rows, columns 16 * lane .. + 15, into registers ----
    // Accumulator slot v holds gate {i, g, f, o}[v]: the transpose-sum below then leaves gate k in lane k.
    half8_t w[4][2];
    {
        const int gate_of_slot[4] = {0, 2, 1, 3};
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const int col = lane * 16 + c * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) w[v][c][e] = (half_t)0.0f;
                if (unit_ok && col < H)  // H % 8 == 0: an 8-wide chunk is entirely inside or outside the row
                    w[v][c] = *reinterpret_cast<const half8_t*>(p.w_hh + ((long)gate_of_slot[v] * H + j) * H + col);
            }
        }
    }
    // Columns at and past H stay zero in both h buffers for the whole kernel.
    for (int i = tid; i < 2 * kSeqMaxH / 8; i += 256) {
        half8_t z;
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = (half_t)0.0f;
        reinterpret_cast<half8_t*>(&hbuf[0][0])[i] = z;
    }
    __syncthreads();

    const bool has_entry = tid < nb;            // lane t fetches the h values of block t
    const int my_gate = lane & 3;               // role of lanes 0..3 after the transpose-sum
    const bool gate_lane = lane < 4 && unit_ok;
    float c_reg = gate_lane ? (float)p.c0[j] : 0.0f;
    bool gave_up = false;

    // The input-projection term does not depend on h: it is fetched two steps ahead, into two registers that
    // alternate between even and odd steps (the step loop is unrolled by two so that no copy of a pending
    // load, and hence no wait for it, is needed at the loop's back edge).
    // Every lane loads (lanes 4..63 repeat the addresses of lanes 0..3, units past H are clamped to H - 1 and
    // steps past the end to the last step): an unconditional load keeps the two registers free of copies.
    const float* xp_ptr = p.xproj + (long)my_gate * H + (unit_ok ? j : H - 1);
    const long xp_step = p.reverse ? -(long)4 * H : (long)4 * H;
    if (p.reverse) xp_ptr += (long)(p.T - 1) * 4 * H;
    float xp_even = xp_ptr[0];
    float xp_odd = xp_ptr[p.T > 1 ? xp_step : 0];

    auto step = [&](const int s, float& xp_slot) __attribute__((always_inline)) {
        const int t = p.reverse ? (p.T - 1 - s) : s;
        half_t* hb = hbuf[s & 1];

        // ---- 1. h_{s-1} of block `tid` into LDS ----
        if (has_entry) {
            half4_t hv;
            if (s == 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) hv[e] = (tid * 4 + e < H) ? p.h0[tid * 4 + e] : (half_t)0.0f;
            } else {
                const unsigned int want = (p.tag_base + (unsigned int)s) & 0xffffu;
                unsigned long long* src =
                    reinterpret_cast<unsigned long long*>(p.hx + ((long)((s - 1) & 1) * nb + tid) * kSeqEntryWords);
                unsigned long long w0 = 0, w1 = 0;
                unsigned int spins = 0;
                while (true) {
                    w0 = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    w1 = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const bool ok = ((unsigned int)(w0 >> 16) & 0xffffu) == want && (unsigned int)(w0 >> 48) == want &&
                                    ((unsigned int)(w1 >> 16) & 0xffffu) == want && (unsigned int)(w1 >> 48) == want;
                    if (ok || gave_up) break;
                    ++spins;
                    if ((spins & 255u) == 0u) {
                        if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                    }
                    if (spins >= p.spin_limit) {
                        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        gave_up = true;
                    }
                }
                hv[0] = __builtin_bit_cast(half_t, (unsigned short)(w0 & 0xffffu));
                hv[1] = __builtin_bit_cast(half_t, (unsigned short)((w0 >> 32) & 0xffffu));
                hv[2] = __builtin_bit_cast(half_t, (unsigned short)(w1 & 0xffffu));
                hv[3] = __builtin_bit_cast(half_t, (unsigned short)((w1 >> 32) & 0xffffu));
            }
            *reinterpret_cast<half4_t*>(hb + tid * 4) = hv;
        }
        __syncthreads();

        // ---- 2. gates: 4 rows x 16 columns per lane, then over the wavefront ----
        const half8_t ha = *reinterpret_cast<const half8_t*>(hb + lane * 16);
        const half8_t hc = *reinterpret_cast<const half8_t*>(hb + lane * 16 + 8);
        float acc[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[v] = dot8(w[v][1], hc, dot8(w[v][0], ha, 0.0f));

        // Transpose-sum: after the two halving exchanges lane l holds slot 2 * (l & 1) + ((l >> 1) & 1) summed
        // over its quad, i.e. gate (l & 3); wave_sum_mod4 then adds the 16 quads.
        const bool b0 = lane & 1, b1 = lane & 2;
        const float a0 = (b0 ? acc[2] : acc[0]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[0] : acc[2]);
        const float a1 = (b0 ? acc[3] : acc[1]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[1] : acc[3]);
        const float a = wave_sum_mod4((b1 ? a1 : a0) + dpp_mov_f32<kDppQuadXor2>(b1 ? a0 : a1)) + xp_slot;
        // The term fetched two steps ago has been consumed: refill the same register for two steps ahead.  (Issued
        // only now so that the old and the new value never live at once, which would cost a copy, and with it a
        // wait for this load and for the stores below, at the loop's back edge.)
        xp_slot = xp_ptr[(long)min(s + 2, p.T - 1) * xp_step];

        // Each of lanes 0..3 activates its own gate: sigmoid for i, f, o and tanh(a) = 2 * sigmoid(2a) - 1 for g.
        const bool is_g = my_gate == 2;
        const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
        const float act = is_g ? 2.0f * sg - 1.0f : sg;
        const float g_i = dpp_mov_f32<0x00>(act);  // quad_perm broadcasts of lanes 0, 1, 2, 3 of the quad
        const float g_f = dpp_mov_f32<0x55>(act);
        const float g_g = dpp_mov_f32<0xAA>(act);
        const float g_o = dpp_mov_f32<0xFF>(act);
        const float c_new = g_f * c_reg + g_i * g_g;
        const half_t h_new = (half_t)(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
        c_reg = c_new;

        // ---- 3. publish ----
        if (lane == 0) {
            const unsigned int hbits = unit_ok ? (unsigned int)__builtin_bit_cast(unsigned short, h_new) : 0u;
            const unsigned int word = hbits | (((p.tag_base + (unsigned int)s + 1u) & 0xffffu) << 16);
            __hip_atomic_store(p.hx + ((long)(s & 1) * nb + blockIdx.x) * kSeqEntryWords + wave, word, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            if (unit_ok) {
                p.y[(long)t * p.y_stride + j] = h_new;
                if (s == p.T - 1) {
                    p.hn[j] = h_new;
                    p.cn[j] = (half_t)c_new;
                }
            }
        }
    };

    int s = 0;
    for (; s + 1 < p.T; s += 2) {
        step(s, xp_even);
        step(s + 1, xp_odd);
    }
    if (s < p.T) step(s, xp_even);
}

}  // namespace pimhip
