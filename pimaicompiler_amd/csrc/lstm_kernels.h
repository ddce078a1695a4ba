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
//   lstm_seq_f16_kernel       one launch for whole sequences of up to four recurrences: every wavefront keeps
//                             the gate rows of its hidden unit and its cell state in registers for all
//                             steps; h_t is exchanged between blocks through flagged words in device memory,
//                             so the per-step cost is one device-scope store/load round trip, not a launch.
#pragma once

#include "device_common.h"
#include "lstm_solo.h"

namespace pimhip
{
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

// ---------------------------------------------------------------------------------------------
// Single step.  One wavefront per hidden unit j: its four gate rows j, H+j, 2H+j, 3H+j.
//   xproj  != nullptr : a = xproj[4H] (fp32, biases included) + W_hh h
//   xproj  == nullptr : a = W_ih x + W_hh h + bsum[4H] (fp32 or nullptr)
// Requirements checked by the launcher: H % 8 == 0, I % 8 == 0, 16-byte aligned pointers.
// c_in_f16 (fp16) is read when non-null, else c_state (fp32); c_state is always written; h_out, and
// hn_f16 / cn_f16 when non-null, receive the new state.
// ---------------------------------------------------------------------------------------------
// The four gate sums of unit j, this lane's share: W_hh[rows of j] . h_prev, and W_ih[rows of j] . x when there is no xproj.
template <bool KEEP>
__device__ __forceinline__ void lstm_step_sums(float (&acc)[4], const half_t* __restrict__ w_ih, const half_t* __restrict__ w_hh,
                                               const float* __restrict__ xproj, const half_t* __restrict__ x,
                                               const half_t* __restrict__ h_prev, int I, int H, int j, int lane)
{
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
                wr[g][0] = load_weight<KEEP>(w0 + g * gstride + c);
                wr[g][1] = load_weight<KEEP>(w0 + g * gstride + c + 64);
            }
            const half8_t h0 = hv[c], h1 = hv[c + 64];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g][1], h1, dot8(wr[g][0], h0, acc[g]));
        }
        for (; c < nchunks; c += 64) {
            half8_t wr[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) wr[g] = load_weight<KEEP>(w0 + g * gstride + c);
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
                wr[g][0] = load_weight<KEEP>(w0 + g * gstride + c);
                wr[g][1] = load_weight<KEEP>(w0 + g * gstride + c + 64);
            }
            const half8_t x0 = xv[c], x1 = xv[c + 64];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g][1], x1, dot8(wr[g][0], x0, acc[g]));
        }
        for (; c < nchunks; c += 64) {
            half8_t wr[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) wr[g] = load_weight<KEEP>(w0 + g * gstride + c);
            const half8_t x0 = xv[c];
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(wr[g], x0, acc[g]);
        }
    }
}

// KEEP: the weights this launch reads are small and the next step's launch reads them again: plain loads (load_weight).
template <int WAVES, bool KEEP>
__global__ __launch_bounds__(WAVES * 64) void lstm_step_f16_kernel(
    const half_t* __restrict__ w_ih, const half_t* __restrict__ w_hh, const float* __restrict__ bsum,
    const float* __restrict__ xproj, const half_t* __restrict__ x, const half_t* __restrict__ h_prev,
    const half_t* __restrict__ c_in_f16, float* __restrict__ c_state, half_t* __restrict__ h_out,
    half_t* __restrict__ hn_f16, half_t* __restrict__ cn_f16, int I, int H)
{
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * WAVES + (threadIdx.x >> 6);
    if (j >= H) return;

    // what the cell needs besides the sums, asked for before the weights: it arrives behind them at no cost, where a load
    // after the reduction is a trip to the L2 of its own at the end of a short kernel
    const int gate = lane & 3;
    float addend = 0.0f;
    if (xproj)
        addend = xproj[(long)gate * H + j];
    else if (bsum)
        addend = bsum[(long)gate * H + j];
    const float c_prev = c_in_f16 ? (float)c_in_f16[j] : c_state[j];

    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    lstm_step_sums<KEEP>(acc, w_ih, w_hh, xproj, x, h_prev, I, H, j, lane);
    // The four gate sums are folded into one reduction: two halving exchanges leave gate l & 3 (i, f, g, o), summed over
    // its quad, in lane l, and the rest of the tree adds the sixteen quads.  Lanes 0..3 of every quad then activate one gate
    // each (sigmoid, and tanh(a) = 2 sigmoid(2a) - 1, on the hardware exp2 and reciprocal: absolute error below 1e-6) and
    // quad broadcasts hand the four gates round: a few dozen instructions where four separate sums and five activations
    // with full divisions in one lane took a tenth of a short launch.
    const bool b0 = lane & 1, b1 = lane & 2;
    const float a0 = (b0 ? acc[1] : acc[0]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[0] : acc[1]);
    const float a1 = (b0 ? acc[3] : acc[2]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[2] : acc[3]);
    float a = (b1 ? a1 : a0) + dpp_mov_f32<kDppQuadXor2>(b1 ? a0 : a1);
    a = wave_sum_mod4(a);
    a += addend;
    const bool is_g = gate == 2;
    const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
    const float act = is_g ? 2.0f * sg - 1.0f : sg;
    const float g_i = dpp_mov_f32<0x00>(act);  // quad_perm broadcasts of lanes 0, 1, 2, 3 of the quad
    const float g_f = dpp_mov_f32<0x55>(act);
    const float g_g = dpp_mov_f32<0xAA>(act);
    const float g_o = dpp_mov_f32<0xFF>(act);
    const float c_new = g_f * c_prev + g_i * g_g;
    const half_t h_new = (half_t)(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
    if (lane == 0) {
        c_state[j] = c_new;
        h_out[j] = h_new;
        if (hn_f16) hn_f16[j] = h_new;
        if (cn_f16) cn_f16[j] = (half_t)c_new;
    }
}

// ---------------------------------------------------------------------------------------------
// Whole sequences in one launch: NC recurrences ("chains") advance together, one super-step at a time.
//
// Two ways to combine chains (template parameter WAVEFRONT):
//   WAVEFRONT = true   chain k is layer k of a unidirectional stack; at super-step tau it computes its time
//                      step tau - k from h of layer k-1 at that time step (its input, multiplied by its W_ih
//                      inside the kernel) and its own h of the step before.  Both were published at super-step
//                      tau - 1, so NC layers cost T + NC - 1 exchanges instead of NC * T.  Only chain 0 takes a
//                      precomputed input projection.
//   WAVEFRONT = false  the chains are independent (the two directions of a bidirectional layer): every chain
//                      takes its own precomputed input projection; chain k runs forward or backward in time.
//
// Grid: NB = ceil(H / UNITS) blocks of UNITS wavefronts (H <= 1024, H % 8 == 0; UNITS = 4, or 8 for a single chain,
// whose entry then still is one 16-byte store and load and whose exchange among half as many blocks is about 0.4 us
// shorter), all resident at once.  Hidden sizes up to 2048 run with COLS = 32 columns of a weight row per lane and eight
// units per block (256 blocks at most), for one layer or the two directions of one (a second layer's W_ih would spill).  The text below is written for UNITS = 4.  Block b owns
// hidden units 4b .. 4b+3 of every chain, one unit per wavefront: wavefront w keeps, per chain, the four W_hh
// gate rows of unit 4b+w (and the four W_ih rows for wavefront chains k > 0) in registers for the whole
// launch (lane l holds columns 16l .. 16l+15 of each row) and the cell states in registers.
//
// A super-step:
//   1. lane t of the block (t < NB) obtains the h values block t published at the previous super-step (four
//      per chain) from the exchange buffer and puts them into LDS; one barrier; every wavefront reads h from LDS;
//   2. per chain: 4 rows x 16 columns of dot products per lane (twice that with W_ih), a transpose-sum over
//      the 64 lanes (6 exchanges) that leaves gate k in lane k, the four activations in parallel in lanes 0..3,
//      the cell update;
//   3. lane 0 of each wavefront stores y and hands its h values to LDS; one barrier; one lane publishes the block's
//      entry with one store per 16 bytes.
//
// Exchange buffer: hx[2][NB] entries of 64 bytes (entries of different blocks do not share a 64-byte segment,
// which measurably shortens the exchange); chain k of block b uses the 8-byte word k of the entry, one fp16 per
// wavefront.  |h| <= 1, so bit 14 of its fp16 pattern is always 0 (a NaN is published as 0) and carries the flag: with g = *g_counter + tau
// counting super-steps over all launches of a plan, super-step g publishes into parity g & 1 with flag bit
// (g >> 1) & 1, i.e. the bit flips every time a slot is rewritten.  A slot can only hold what was published two
// super-steps earlier or the current values (publishing g + 2 needs the words of g + 1 from all blocks, which
// they publish only after reading g), so one bit tells them apart; every fp16 carries it, so a reader validates
// each 8-byte word on its own.  A block gathers its values in LDS and publishes them with ONE store (8 bytes for
// one chain, 16 for two); a waiting lane reads a block's entry with ONE load of the same size.  The round trip of
// that pair through the memory side is the cost of a super-step: measured at 256 blocks, every further load per
// poll and every further store per block adds about 0.3 us.  The buffer is zero when g = 2, the value
// the host initialises the counter with; every launch writes every fp16 of every entry in every super-step, so the
// sequence of flag bits per slot stays alternating across launches.  After a time-out the host clears the buffer and
// sets the counter back to 2.
//
// Every wait is bounded: after `spin_limit` polls (or one second) a lane raises *abort_flag and stops waiting; lanes poll
// the flag every 256 spins and stop waiting once it is set.  A block in which a lane stopped waiting publishes nothing
// from then on (so that no other block takes values for real that were computed from stale ones), leaves the loop of
// super-steps and computes its chains by itself (lstm_solo.h): slower, but the call's result is what it would have been.
// The abort word stays up: later launches of the plan start in that self-sufficient mode until the host has re-initialised
// the exchange buffer.
// ---------------------------------------------------------------------------------------------
static constexpr int kSeqUnits = 4;        // hidden units per block, one per wavefront
static constexpr int kSeqMaxH = 1024;      // 64 lanes x 16 columns
static constexpr int kSeqMaxHWide = 2048;  // 64 lanes x 32 columns (eight units per block; one layer, or the two directions of one)
static constexpr int kSeqEntryWords = 16;  // 32-bit words between the entries of consecutive blocks (64 bytes)
static constexpr int kSeqMaxT = 1 << 30;    // super-steps per launch (the counters are 32-bit)
static constexpr int kSeqMaxChains = 4;

struct LstmSeqChain {
    const half_t* w_hh;   // [4H, H]
    const half_t* w_ih;   // [4H, H]: wavefront chains k > 0 only
    const float* xproj;   // [T, 4H] fp32 with biases: chain 0, and every chain when not in wavefront mode
    const float* bsum;    // [4H] fp32 b_ih + b_hh: wavefront chains k > 0 only
    const half_t* h0;     // [H]
    const half_t* c0;     // [H]
    half_t* y;            // row t at y + t * y_stride; may be null (inner layers of a wavefront)
    half_t* hn;           // [H]
    half_t* cn;           // [H]
    int reverse;          // 1: this chain processes t = T-1 .. 0 (not in wavefront mode)
};

struct LstmSeqArgs {
    LstmSeqChain chain[kSeqMaxChains];
    unsigned int* hx;          // [2][NB][kSeqEntryWords]; zero when *g_counter == 2
    unsigned int* abort_flag;  // set to 1 when a wait gives up; polled by the other waiting lanes
    unsigned int* abort_host;  // host-visible word set at the same time (what the host reads afterwards)
    long y_stride;             // elements between consecutive time steps of y
    int H;
    int T;
    unsigned int* g_counter;   // device word: super-steps this buffer has seen so far, plus 2; advanced by the kernel
    unsigned int spin_limit;
};

template <int NC, bool WAVEFRONT, int UNITS = kSeqUnits, int COLS = 16>
__global__ __launch_bounds__(64 * UNITS) void lstm_seq_f16_kernel(LstmSeqArgs p)
{
    static_assert(UNITS == 4 || UNITS == 8, "one or two 8-byte words per chain and block");
    static_assert(COLS == 16 || COLS == 32, "columns of a weight row per lane");
    constexpr int MAXH = 64 * COLS;  // widest hidden state this instantiation takes
    constexpr int CH = COLS / 8;     // 16-byte pieces of a weight row per lane
    static_assert(MAXH <= 64 * UNITS * UNITS, "lane t of a block fetches the entry of block t");
    constexpr int WPC = UNITS / 4;  // 8-byte words per chain in an entry
    constexpr int NW = NC * WPC;    // 8-byte words of an entry that are in use
    static_assert(NC >= 1 && NC <= kSeqMaxChains && 2 * NW <= kSeqEntryWords, "an entry is 64 bytes");
    __shared__ __align__(16) half_t hbuf[2][NC][MAXH];       // published h per chain, double buffered by parity
    __shared__ __align__(16) unsigned short pub[NC][UNITS];  // this block's next entry: chain k, wavefront w
    __shared__ int block_gave_up;                            // set by a lane whose wait gave up; read by all after the step's first barrier

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int H = p.H;
    const int T = p.T;
    const int nb = gridDim.x;
    const int j = blockIdx.x * UNITS + wave;  // this wavefront's hidden unit
    const bool unit_ok = j < H;
    const int n_super = WAVEFRONT ? T + NC - 1 : T;
    // The count of super-steps lives in device memory and is advanced by the kernel itself (last statement), so that a
    // launch carries no host-side state and replays from a graph like any other.  Device-scope load: the previous
    // launch stored it from another XCD.  The value is first needed when super-step 0 publishes.
    const unsigned int g_base = __builtin_amdgcn_readfirstlane(
        __hip_atomic_load(p.g_counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    // A wait of an earlier launch gave up and the host has not re-initialised the exchange buffer since (it may hold that
    // launch's values): nothing is exchanged, every block computes its chains by itself.
    const bool poisoned = __builtin_amdgcn_readfirstlane(__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) != 0u;
    if (tid == 0) block_gave_up = poisoned ? 1 : 0;

    // ---- weights into registers: per chain the four gate rows of unit j, columns 16 * lane .. + 15 ----
    // Accumulator slot v holds gate {i, g, f, o}[v]: the transpose-sum below then leaves gate k in lane k.
    half8_t w_hh[NC][4][CH];
    half8_t w_ih[WAVEFRONT ? NC : 1][4][CH];  // entry 0 unused
    {
        const int gate_of_slot[4] = {0, 2, 1, 3};
        half8_t zero;
#pragma unroll
        for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;
#pragma unroll
        for (int k = 0; k < NC; ++k) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const int col = lane * COLS + c * 8;
                    const bool ok = unit_ok && col < H;  // H % 8 == 0: a chunk is entirely inside or outside the row
                    const long off = ((long)gate_of_slot[v] * H + j) * H + col;
                    w_hh[k][v][c] = ok ? *reinterpret_cast<const half8_t*>(p.chain[k].w_hh + off) : zero;
                    if (WAVEFRONT && k > 0) w_ih[k][v][c] = ok ? *reinterpret_cast<const half8_t*>(p.chain[k].w_ih + off) : zero;
                }
            }
        }
        // Columns at and past H stay zero in all h buffers for the whole kernel.
        for (int i = tid; i < 2 * NC * MAXH / 8; i += 64 * UNITS) reinterpret_cast<half8_t*>(&hbuf[0][0][0])[i] = zero;
    }
    __syncthreads();

    const bool has_entry = tid < nb;  // lane t fetches what block t published
    const int my_gate = lane & 3;     // role of lanes 0..3 after the transpose-sum
    const int jc = unit_ok ? j : H - 1;
    float c_reg[NC];
    float bias_reg[NC];               // wavefront chains k > 0: b_ih + b_hh of (gate my_gate, unit j)
    const float* xp_ptr[NC];
    long xp_step[NC];
    float xp_even[NC], xp_odd[NC];
#pragma unroll
    for (int k = 0; k < NC; ++k) {
        c_reg[k] = (float)p.chain[k].c0[jc];
        bias_reg[k] = 0.0f;
        xp_ptr[k] = nullptr;
        xp_step[k] = 0;
        xp_even[k] = xp_odd[k] = 0.0f;
        if (WAVEFRONT && k > 0) {
            bias_reg[k] = p.chain[k].bsum[(long)my_gate * H + jc];
        } else {
            // The input-projection term does not depend on h: it is fetched two steps ahead into two registers
            // that alternate between even and odd steps (the loop is unrolled by two).  Every lane loads (lanes
            // 4..63 repeat the addresses of lanes 0..3; steps past the end are clamped to the last one): an
            // unconditional load keeps the registers free of copies, and with them of waits at the back edge.
            const bool rev = p.chain[k].reverse != 0;
            xp_ptr[k] = p.chain[k].xproj + (long)my_gate * H + jc + (rev ? (long)(T - 1) * 4 * H : 0);
            xp_step[k] = rev ? -(long)4 * H : (long)4 * H;
            xp_even[k] = xp_ptr[k][0];
            xp_odd[k] = xp_ptr[k][T > 1 ? xp_step[k] : 0];
        }
    }
    bool gave_up = false;

    bool alone = poisoned;  // the block has to go on by itself (a wait gave up)
    auto super_step = [&](const int tau, float (&xp_slot)[NC]) __attribute__((always_inline)) {
        half_t(*hb)[MAXH] = hbuf[tau & 1];

        // ---- 1. what block `tid` published at super-step tau - 1 (or the initial state) into LDS ----
        if (has_entry) {
            unsigned long long words[NW];  // words k * WPC ..: the UNITS fp16 of chain k published by block `tid`
#pragma unroll
            for (int k = 0; k < NW; ++k) words[k] = 0ull;
            if (tau > 0) {
                const unsigned int gp = g_base + (unsigned int)tau - 1u;  // the super-step whose values are awaited
                const unsigned long long want = ((gp >> 1) & 1u) ? 0x4000400040004000ull : 0ull;
                const unsigned long long* src =
                    reinterpret_cast<const unsigned long long*>(p.hx + ((long)(gp & 1u) * nb + tid) * kSeqEntryWords);
                unsigned int spins = 0;
                unsigned long long t_first = 0ull;
                while (true) {
                    bool ok = true;
#pragma unroll
                    for (int k = 0; k + 1 < NW; k += 2) load16_device_scope(src + k, words[k], words[k + 1]);
                    if (NW & 1)
                        words[NW - 1] = __hip_atomic_load(const_cast<unsigned long long*>(src) + (NW - 1), __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int k = 0; k < NW; ++k) ok = ok && (words[k] & 0x4000400040004000ull) == want;
                    if (ok || gave_up) break;
                    ++spins;
                    if ((spins & 255u) == 0u) {
                        if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                        if (wait_clock_expired(spins, t_first)) spins = 0xffffffffu;  // gives up below
                    }
                    if (spins >= p.spin_limit) {
                        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        gave_up = true;
                    }
                    if (gave_up) block_gave_up = 1;  // (its own wait or another block's: this block's h would be made from stale values)
                }
            }
#pragma unroll
            for (int k = 0; k < NC; ++k) {
                const int s_k = WAVEFRONT ? tau - k : tau;  // the time step chain k computes now
#pragma unroll
                for (int q = 0; q < WPC; ++q) {
                    half4_t hv;
                    if (s_k == 0) {
                        // First step of this chain: its previous h is the caller's initial state.
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int u = tid * UNITS + q * 4 + e;
                            hv[e] = (u < H) ? p.chain[k].h0[u] : (half_t)0.0f;
                        }
                    } else {
                        // Units 4q .. 4q+3 of chain k in block `tid`, flag bit removed.
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            hv[e] = __builtin_bit_cast(half_t, (unsigned short)((words[k * WPC + q] >> (16 * e)) & 0xbfffu));
                    }
                    *reinterpret_cast<half4_t*>(&hb[k][tid * UNITS + q * 4]) = hv;
                }
            }
        }
        __syncthreads();
        // Written only in front of this barrier: every thread reads the same value, and the block leaves together.  Asked
        // for here, with the reads of h, and looked at where the block would publish: the step's arithmetic does not wait
        // for it (a step that should not have been made is made on stale values and dropped).
        const int gave_up_in_this_step = __builtin_amdgcn_readfirstlane(block_gave_up);

        // ---- 2. gates of all chains ----
        // Written without branches and phase by phase over the chains, so that the chains' dependency chains
        // (LDS read, dot products, six exchange steps, exp / rcp) overlap instead of running one after another.  A
        // chain that has not started or has finished computes on whatever its buffer holds; the result is dropped.
        float acc[NC][4];
#pragma unroll
        for (int k = 0; k < NC; ++k) {
            half8_t hv[CH];
#pragma unroll
            for (int c = 0; c < CH; ++c) hv[c] = *reinterpret_cast<const half8_t*>(&hb[k][lane * COLS + c * 8]);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                acc[k][v] = 0.0f;
#pragma unroll
                for (int c = 0; c < CH; ++c) acc[k][v] = dot8(w_hh[k][v][c], hv[c], acc[k][v]);
            }
            if (WAVEFRONT && k > 0) {
                // Input of layer k at its time step: h of layer k - 1 at the same time step, published one
                // super-step ago, which is what chain k - 1's buffer holds now.
                half8_t xv[CH];
#pragma unroll
                for (int c = 0; c < CH; ++c) xv[c] = *reinterpret_cast<const half8_t*>(&hb[k - 1][lane * COLS + c * 8]);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
#pragma unroll
                    for (int c = 0; c < CH; ++c) acc[k][v] = dot8(w_ih[k][v][c], xv[c], acc[k][v]);
                }
            }
        }

        // Transpose-sum: after the two halving exchanges lane l holds slot 2 * (l & 1) + ((l >> 1) & 1) summed over
        // its quad, i.e. gate (l & 3); wave_sum_mod4 then adds the 16 quads.
        const bool b0 = lane & 1, b1 = lane & 2;
        float a[NC];
#pragma unroll
        for (int k = 0; k < NC; ++k) {
            const float a0 = (b0 ? acc[k][2] : acc[k][0]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[k][0] : acc[k][2]);
            const float a1 = (b0 ? acc[k][3] : acc[k][1]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[k][1] : acc[k][3]);
            a[k] = (b1 ? a1 : a0) + dpp_mov_f32<kDppQuadXor2>(b1 ? a0 : a1);
        }
#pragma unroll
        for (int k = 0; k < NC; ++k) a[k] = wave_sum_mod4(a[k]);

        half_t h_new[NC];
        bool h_is_number[NC];
        float c_out[NC];
        const bool is_g = my_gate == 2;
#pragma unroll
        for (int k = 0; k < NC; ++k) {
            const int s_k = WAVEFRONT ? tau - k : tau;
            const bool active = s_k >= 0 && s_k < T;
            if (WAVEFRONT && k > 0) {
                a[k] += bias_reg[k];
            } else {
                a[k] += xp_slot[k];
                // The term fetched two steps ago has been consumed: refill the same register for two steps ahead.
                // (Issued only now so that the old and the new value never live at once, which would cost a copy,
                // and with it a wait for this load and for the stores below, at the loop's back edge.)
                xp_slot[k] = xp_ptr[k][(long)max(0, min(s_k + 2, T - 1)) * xp_step[k]];
            }
            // Each of lanes 0..3 activates its own gate: sigmoid for i, f, o and tanh(a) = 2 * sigmoid(2a) - 1 for g.
            const float sg = fast_sigmoid_f32(is_g ? 2.0f * a[k] : a[k]);
            const float act = is_g ? 2.0f * sg - 1.0f : sg;
            const float g_i = dpp_mov_f32<0x00>(act);  // quad_perm broadcasts of lanes 0, 1, 2, 3 of the quad
            const float g_f = dpp_mov_f32<0x55>(act);
            const float g_g = dpp_mov_f32<0xAA>(act);
            const float g_o = dpp_mov_f32<0xFF>(act);
            const float c_new = g_f * c_reg[k] + g_i * g_g;
            // h is NaN exactly when c_new or the output gate is; known here, before the tanh, off the critical path
            h_is_number[k] = (c_new == c_new) && (g_o == g_o);
            const half_t h = (half_t)(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
            h_new[k] = active ? h : (half_t)0.0f;
            c_reg[k] = active ? c_new : c_reg[k];
            c_out[k] = c_new;
        }

        // ---- 3. outputs, then publish ----
        // The block's values are gathered in LDS and published by ONE lane with ONE store per 16 bytes: the time
        // until every block has seen a super-step grows by about 0.3 us with every further store per block.
        if (lane == 0) {
            const unsigned int flag = (((g_base + (unsigned int)tau) >> 1) & 1u) << 14;
#pragma unroll
            for (int k = 0; k < NC; ++k) {
                // A NaN (from non-finite inputs or weights) has bit 14 set and cannot travel with the flag: y, hn and
                // cn below still receive it, the exchange carries 0 for this unit instead of making every reader wait
                // for a flag that never matches.
                const unsigned int hbits = (unit_ok && h_is_number[k]) ? (unsigned int)__builtin_bit_cast(unsigned short, h_new[k]) : 0u;
                pub[k][wave] = (unsigned short)(hbits | flag);
            }
            if (unit_ok) {
#pragma unroll
                for (int k = 0; k < NC; ++k) {
                    const int s_k = WAVEFRONT ? tau - k : tau;
                    if (s_k < 0 || s_k >= T) continue;
                    const int t = p.chain[k].reverse ? (T - 1 - s_k) : s_k;
                    if (p.chain[k].y) p.chain[k].y[(long)t * p.y_stride + j] = h_new[k];
                    if (s_k == T - 1) {
                        p.chain[k].hn[j] = h_new[k];
                        p.chain[k].cn[j] = (half_t)c_out[k];
                    }
                }
            }
        }
        __syncthreads();
        alone = gave_up_in_this_step != 0;
        if (tid == 0 && !alone) {
            const unsigned int g = g_base + (unsigned int)tau;
            unsigned long long* dst = reinterpret_cast<unsigned long long*>(p.hx + ((long)(g & 1u) * nb + blockIdx.x) * kSeqEntryWords);
            const unsigned long long* src = reinterpret_cast<const unsigned long long*>(&pub[0][0]);
#pragma unroll
            for (int k = 0; k + 1 < NW; k += 2) store16_device_scope(dst + k, src[k], src[k + 1]);
            if (NW & 1) __hip_atomic_store(dst + (NW - 1), src[NW - 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    int tau = 0;
    for (; !alone && tau + 1 < n_super; tau += 2) {
        super_step(tau, xp_even);
        if (!alone) super_step(tau + 1, xp_odd);
    }
    if (!alone && tau < n_super) super_step(tau, xp_even);
    if (alone) {
        // ---- self-sufficient: this block's units of every chain, from the call's inputs, by this block alone ----
        SoloStack st;
        st.y_stride = p.y_stride;
        st.H = H;
        st.T = T;
        st.res_in0 = nullptr;
        const int u_begin = min(blockIdx.x * UNITS, H), u_end = min(u_begin + UNITS, H);
        auto layer_of = [&](int k) {
            SoloLayer ly;
            ly.w_hh = p.chain[k].w_hh;
            ly.w_ih = nullptr;
            ly.bsum = nullptr;
            ly.h0 = p.chain[k].h0;
            ly.c0 = p.chain[k].c0;
            ly.y = p.chain[k].y;
            ly.hn = p.chain[k].hn;
            ly.cn = p.chain[k].cn;
            ly.residual = 0;
            ly.u_begin = u_begin;
            ly.u_end = u_end;
            return ly;
        };
        if (WAVEFRONT) {
            st.n = NC;
            st.xproj = p.chain[0].xproj;
            st.reverse = 0;
#pragma unroll
            for (int k = 0; k < NC; ++k) {
                st.layer[k] = layer_of(k);
                if (k > 0) {
                    st.layer[k].w_ih = p.chain[k].w_ih;
                    st.layer[k].bsum = p.chain[k].bsum;
                }
            }
            lstm_solo_stack<64 * UNITS, NC, MAXH>(st);
        } else {
            for (int k = 0; k < NC; ++k) {  // independent chains, one after the other
                st.n = 1;
                st.xproj = p.chain[k].xproj;
                st.reverse = p.chain[k].reverse;
                st.layer[0] = layer_of(k);
                lstm_solo_stack<64 * UNITS, 1, MAXH>(st);
            }
        }
    }
    // Block 0 has finished its last super-step, for which (n_super >= 2, the launcher's condition) it needed what every
    // block published one super-step earlier: every block has read the counter by now.  The next launch reads it after
    // this one has ended.
    if (blockIdx.x == 0 && tid == 0)
        __hip_atomic_store(p.g_counter, g_base + (unsigned int)n_super, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
