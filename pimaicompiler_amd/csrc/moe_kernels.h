// One launch for a token's pass through a top-1 mixture-of-experts feed-forward block (gfx950, batch 1, fp16 storage,
// fp32 sums):
//
//     logits = W_r . x (+ b_r)          e = argmax(logits)          (the first maximum, on the logits rounded to fp16)
//     hidden = act(W1[e] . x + b1[e])                               (rounded to fp16, as the tensor between the two products is)
//     y      = W2[e] . hidden + b2[e]   (optionally times softmax(logits)[e])
//
// The reference runs this as separate operators (the router and the two products through customAtenAddmm / atenLinear,
// runtime/source/executor/op_executor/aten_ops.cpp:609-758 and :304-307) with the choice of the expert made on the host
// in between, which costs a stream synchronisation and a read-back per token.  Here the choice never leaves the GPU:
// every block computes the router's few rows itself, reads its rows of the chosen expert's first matrix, publishes its
// slice of `hidden` and, once it has everybody's, multiplies its rows of the second matrix, which are already in
// registers by then.
//
// Grid: kMoeBlocks blocks of four wavefronts, all resident at once.  Block b owns rows [b * rpb1, (b + 1) * rpb1) of W1
// and rows [b * rpb2, (b + 1) * rpb2) of W2; local row i belongs to wavefront i % 4, whose lanes stride over the row's
// 16-byte pieces.
//
// Exchange: hx[2][blocks] entries of 64 bytes; a block's hidden values (at most 16) in the first 32 bytes as four 8-byte
// words.  An empty word is all ones, which no four fp16 values written here can be (a NaN is written as 0x7e00).  The
// two sets alternate by the launch count g (a device word read at the start and advanced by block 0 at the end): a
// launch uses set g & 1 and marks its own entry of the other set empty for the launch after it.  Every wait is bounded:
// after `spin_limit` polls a lane raises the abort flags, all lanes stop waiting, the kernel runs to its end with
// undefined results and the host reports a time-out and refills both sets before the next launch.
#pragma once

#include "device_common.h"

namespace pimhip
{

constexpr int kMoeThreads = 256;
constexpr int kMoeWaves = kMoeThreads / 64;
constexpr int kMoeBlocks = 256;
constexpr int kMoeMaxExperts = 64;
constexpr int kMoeMaxModel = 2048;                    // d_model: at most four 16-byte pieces of a row per lane
constexpr int kMoeMaxFf = 4096;                       // d_ff: at most eight 16-byte pieces of a W2 row per lane
constexpr int kMoeXC = kMoeMaxModel / 8 / 64;
constexpr int kMoeFC = kMoeMaxFf / 8 / 64;
constexpr int kMoeRows1 = kMoeMaxFf / kMoeBlocks / kMoeWaves;     // W1 rows per wavefront: 4
constexpr int kMoeRows2 = kMoeMaxModel / kMoeBlocks / kMoeWaves;  // W2 rows per wavefront: 2
constexpr int kMoeEntryWords = 8;                     // 8-byte words per entry (64 bytes); the first four carry values
constexpr unsigned long long kMoeEmpty = ~0ull;
static_assert(kMoeBlocks <= kMoeThreads, "thread t of a block polls block t's entry");
static_assert(kMoeRows1 * kMoeWaves <= 16, "a block's hidden values fit the four 8-byte words of its entry");

struct MoeStepArgs {
    const half_t* x;                 // [d_model]
    const half_t* router_w;          // [E, d_model]
    const half_t* router_b;          // [E] or null
    const half_t* const* tables;     // device array [4][E]: W1[e] ([d_ff, d_model]), b1[e] or null, W2[e] ([d_model, d_ff]), b2[e] or null
    half_t* y;                       // [d_model]
    half_t* router_logits;           // [E] or null
    int* expert;                     // [1] or null
    unsigned long long* hx;          // [2][kMoeBlocks][kMoeEntryWords]
    unsigned int* g_counter;
    unsigned int* abort_flag;
    unsigned int* abort_host;
    int d_model, d_ff, E, act, scale_by_prob;
    int rpb1, rpb2;                  // rows of W1 / W2 per block
    unsigned int spin_limit;
};

__global__ __launch_bounds__(kMoeThreads) void moe_ffn_step_f16_kernel(MoeStepArgs p)
{
    __shared__ __align__(16) half_t hidden[kMoeMaxFf];
    __shared__ float logit_s[kMoeMaxExperts];
    __shared__ const half_t* table_s[4][kMoeMaxExperts];
    __shared__ __align__(8) unsigned short mine[16];  // this block's hidden values (bits), zeros where it has no row

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x, nb = gridDim.x;
    const int nx = p.d_model >> 3, nf = p.d_ff >> 3;
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;

    const unsigned int g = __hip_atomic_load(p.g_counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned int set = g & 1u;
    // this block's entry of the other set is empty for the next launch (nobody reads that set during this one)
    if (tid < kMoeEntryWords)
        __hip_atomic_store(p.hx + ((long)(set ^ 1u) * nb + b) * kMoeEntryWords + tid, kMoeEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid < 16) mine[tid] = 0;
    // the experts' pointers, while the router's rows travel
    for (int i = tid; i < 4 * p.E; i += kMoeThreads) table_s[i / p.E][i % p.E] = p.tables[i];

    // ---- the token, then the router: every block computes all E logits ----
    half8_t xr[kMoeXC];
    const half8_t* x8 = reinterpret_cast<const half8_t*>(p.x);
#pragma unroll
    for (int k = 0; k < kMoeXC; ++k) xr[k] = (lane + 64 * k < nx) ? x8[lane + 64 * k] : zero8;
    // (two experts per wavefront and pass: all their loads are in flight together, one round trip for E <= 8)
    for (int e0 = wave; e0 < p.E; e0 += 2 * kMoeWaves) {
        const int e1 = e0 + kMoeWaves;
        const half8_t* w8a = reinterpret_cast<const half8_t*>(p.router_w) + (long)e0 * nx;
        const half8_t* w8b = reinterpret_cast<const half8_t*>(p.router_w) + (long)(e1 < p.E ? e1 : e0) * nx;
        half8_t ra[kMoeXC], rb[kMoeXC];
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k) {
            const int c = min(lane + 64 * k, nx - 1);
            ra[k] = w8a[c];
            rb[k] = w8b[c];
        }
        float sa = 0.0f, sb = 0.0f;
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k) {
            if (lane + 64 * k < nx) {
                sa = dot8(ra[k], xr[k], sa);
                sb = dot8(rb[k], xr[k], sb);
            }
        }
        sa = wave_sum(sa);
        sb = wave_sum(sb);
        if (lane == 0) {
            if (p.router_b) sa += (float)p.router_b[e0];
            logit_s[e0] = (float)(half_t)sa;
            if (e1 < p.E) {
                if (p.router_b) sb += (float)p.router_b[e1];
                logit_s[e1] = (float)(half_t)sb;
            }
        }
    }
    __syncthreads();
    // argmax over the E <= 64 logits, one per lane: the first maximum; a NaN counts as the largest value, as in at::argmax
    const float mine_l = lane < p.E ? logit_s[lane] : -INFINITY;
    const bool is_nan = mine_l != mine_l;
    const unsigned long long nan_mask = __ballot(is_nan);
    float bv = is_nan ? -INFINITY : mine_l;
    bv = fmaxf(bv, dpp_f32<kDppQuadXor1>(bv));
    bv = fmaxf(bv, dpp_f32<kDppQuadXor2>(bv));
    bv = fmaxf(bv, dpp_f32<kDppRowHalfMirror>(bv));
    bv = fmaxf(bv, dpp_f32<kDppRowMirror>(bv));
    bv = fmaxf(bv, __shfl_xor(bv, 16, kWave));
    bv = fmaxf(bv, __shfl_xor(bv, 32, kWave));
    const unsigned long long max_mask = __ballot(lane < p.E && mine_l == bv);
    const int best = nan_mask ? __builtin_ctzll(nan_mask) : __builtin_ctzll(max_mask);
    float scale = 1.0f;
    if (p.scale_by_prob) {
        const float ex = lane < p.E ? __expf(mine_l - bv) : 0.0f;
        scale = 1.0f / wave_sum(ex);
    }
    if (b == 0) {
        if (tid == 0 && p.expert) p.expert[0] = best;
        if (tid < p.E && p.router_logits) p.router_logits[tid] = (half_t)logit_s[tid];
    }
    const half8_t* w1 = reinterpret_cast<const half8_t*>(table_s[0][best]);
    const half_t* b1 = table_s[1][best];
    const half8_t* w2 = reinterpret_cast<const half8_t*>(table_s[2][best]);
    const half_t* b2 = table_s[3][best];

    // ---- hidden = act(W1[e] . x + b1[e]): this block's rows ----
    half8_t w1r[kMoeRows1][kMoeXC];
#pragma unroll
    for (int s = 0; s < kMoeRows1; ++s) {
        const int r = min(b * p.rpb1 + wave + kMoeWaves * s, p.d_ff - 1);  // (rows this block does not own are loaded and dropped)
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k) w1r[s][k] = load_stream(w1 + (long)r * nx + min(lane + 64 * k, nx - 1));
    }
#pragma unroll
    for (int s = 0; s < kMoeRows1; ++s) {
        const int i = wave + kMoeWaves * s;
        const int r = b * p.rpb1 + i;
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k)
            if (lane + 64 * k < nx) a = dot8(w1r[s][k], xr[k], a);
        a = wave_sum(a);
        if (lane == 0 && i < p.rpb1 && r < p.d_ff) {
            if (b1) a += (float)b1[r];
            if (p.act == 1) a = fmaxf(a, 0.0f);
            unsigned short bits = __builtin_bit_cast(unsigned short, (half_t)a);
            if (a != a) bits = 0x7e00u;
            mine[i] = bits;
        }
    }
    __syncthreads();
    if (tid < 4) {
        const unsigned long long word = *reinterpret_cast<const unsigned long long*>(&mine[4 * tid]);
        __hip_atomic_store(p.hx + ((long)set * nb + b) * kMoeEntryWords + tid, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // ---- everybody's hidden values: thread t takes block t's entry ----
    half8_t w2r[kMoeRows2][kMoeFC];
    {
        const int first = tid * p.rpb1;               // block tid's first row
        const int rows = min(p.rpb1, p.d_ff - first);  // <= 0: that block has no row
        // A block without rows publishes zeros and is waited for all the same: block 0 advances the launch count at its end,
        // and no block may still be on its way to reading it then.
        const int words = tid < nb ? (rows > 0 ? (rows + 3) >> 2 : 1) : 0;
        const unsigned long long* slot = p.hx + ((long)set * nb + tid) * kMoeEntryWords;
        unsigned long long got[4] = {0ull, 0ull, 0ull, 0ull};
        auto poll = [&]() {
            bool ok = true;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                if (w < words) {
                    got[w] = __hip_atomic_load(const_cast<unsigned long long*>(slot) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ok = ok && got[w] != kMoeEmpty;
                }
            }
            return ok;
        };
        // This block's rows of W2[e] are asked for behind the store and in front of the first look: they travel while the
        // hidden values do.  (Measured on MI355X, 768 / 3072 / 8 experts: 8.3 us per step this way; asked for together
        // with W1's rows they delay every block's hidden values, 8.7 us; asked for behind the first look they put a whole
        // round trip in front of the second, 9.1 us.)
#pragma unroll
        for (int s = 0; s < kMoeRows2; ++s) {
            const int r = min(b * p.rpb2 + wave + kMoeWaves * s, p.d_model - 1);
#pragma unroll
            for (int k = 0; k < kMoeFC; ++k) w2r[s][k] = load_stream(w2 + (long)r * nf + min(lane + 64 * k, nf - 1));
        }
        bool ok = poll();
        unsigned int spins = 0;
        unsigned long long t_first = 0ull;
        while (!ok) {
            if (spins > 0u && (spins & 255u) == 0u) {
                if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) break;
                if (wait_clock_expired(spins, t_first)) spins = 0xffffffffu;  // gives up below
            }
            if (spins >= p.spin_limit) {  // (with a limit of 0 a lane whose first look failed gives up without another)
                __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                break;
            }
            if (spins != 0xffffffffu) ++spins;
            ok = poll();
        }
        for (int i = 0; i < rows && tid < nb; ++i)
            hidden[first + i] = __builtin_bit_cast(half_t, (unsigned short)(got[i >> 2] >> (16 * (i & 3))));
    }
    __syncthreads();

    // ---- y = W2[e] . hidden + b2[e] ----
    half8_t hr[kMoeFC];
#pragma unroll
    for (int k = 0; k < kMoeFC; ++k) hr[k] = (lane + 64 * k < nf) ? *reinterpret_cast<const half8_t*>(&hidden[(lane + 64 * k) * 8]) : zero8;
#pragma unroll
    for (int s = 0; s < kMoeRows2; ++s) {
        const int i = wave + kMoeWaves * s;
        const int r = b * p.rpb2 + i;
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kMoeFC; ++k)
            if (lane + 64 * k < nf) a = dot8(w2r[s][k], hr[k], a);
        a = wave_sum(a);
        if (lane == 0 && i < p.rpb2 && r < p.d_model) {
            if (b2) a += (float)b2[r];
            p.y[r] = (half_t)(a * scale);
        }
    }
    if (b == 0 && tid == 0) __hip_atomic_store(p.g_counter, g + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
