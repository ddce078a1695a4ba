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
// Grid: `blocks` blocks of eight wavefronts, all resident at once.  `hidden` travels as 16-byte words of eight values;
// block b makes words [b * wpb, (b + 1) * wpb) (wpb = 1 or 2: at most 256 blocks make the at most 512 words), i.e.
// rows 8 * wpb * b .. of W1, wavefront w the rows w * wpb .. of those.  Of W2 block b owns rows [b * rpb2, (b + 1) * rpb2),
// rpb2 <= 8, one row per wavefront.
//
// What bounds the step is not bandwidth (9.4 MB) but a chain of dependent round trips: token and router rows, the expert's
// W1 rows, the all-to-all of `hidden`, the store of y.  So nothing else may stand in that chain: the launch count (which
// says which set of exchange slots this launch uses) is a device-scope load and is asked for behind the router's cached
// loads, not in front of them; the
// slots of the other set are emptied at the very end; a lane that waits looks at ONE 16-byte word of ONE producer per poll
// (a poll round over all blocks gets slower with every further load per lane); the row of W2 is asked for right behind
// the rows of W1 and has arrived when the hidden values have.
//
// Exchange: hx[2][blocks] entries of 64 bytes, a block's words in the first 16 * wpb bytes.  An empty 8-byte half is all
// ones, which no four fp16 values written here can be (a NaN is written as 0x7e00).  The two sets alternate by the launch
// count g (a device word read at the start): a launch uses set g & 1 and marks its own entry of the other set empty for the
// launch after it.  Where every block publishes a word, block 0 advances the count at its end: it has seen everybody's word
// by then, so everybody has read the count.  A block that publishes nothing could start so late that it reads the count
// after block 0 has advanced it, and would look into the wrong set; grids with such blocks (d_model > d_ff / 2) keep one copy
// of the count per block, each in a line of its own, read and advanced by its block (0.3 us slower per step).
//
// A wait that gives up does not leave the result undefined.  Every wait is bounded (`spin_limit` polls, one second); a block
// in which a lane gave up computes every hidden value itself from W1[e] (no other block is needed for that: it is only
// slower, a few tens of microseconds) and goes on.  It raises the plan's abort word, which stays up: every later launch
// starts in that self-sufficient mode (the exchange slots may hold values of the launch that was cut short) until the
// host has refilled the slots and cleared the word.
#pragma once

#include "device_common.h"

namespace pimhip
{

constexpr int kMoeThreads = 512;
constexpr int kMoeWaves = kMoeThreads / 64;
constexpr int kMoeMaxBlocks = 256;
constexpr int kMoeMaxExperts = 64;
constexpr int kMoeMaxModel = 2048;                    // d_model: at most four 16-byte pieces of a row per lane
constexpr int kMoeMaxFf = 4096;                       // d_ff: at most 512 words of eight hidden values, one per thread
constexpr int kMoeXC = kMoeMaxModel / 8 / 64;         // 16-byte pieces of a W1 row per lane
constexpr int kMoeFC = kMoeMaxFf / 8 / 64;            // 16-byte pieces of a W2 row per lane
constexpr int kMoeMaxWordsPerBlock = 2;               // wpb
constexpr int kMoeMaxRows2 = kMoeWaves;               // W2 rows per block: one per wavefront
constexpr int kMoeEntryWords = 8;                     // 8-byte words per entry (64 bytes); the first 2 * wpb carry values
constexpr unsigned long long kMoeEmpty = ~0ull;
constexpr int kMoeCounterStride = 16;                // 32-bit words between the blocks' copies of the launch count: a 64-byte line each
static_assert(kMoeMaxFf / 8 <= kMoeThreads, "thread t of a block polls word t");
static_assert(kMoeMaxWordsPerBlock * kMoeMaxBlocks * 8 >= kMoeMaxFf, "every hidden value has a producer");
static_assert(2 * kMoeMaxWordsPerBlock <= kMoeEntryWords, "a block's words fit its entry");

struct MoeStepArgs {
    const half_t* x;                 // [d_model]
    const half_t* router_w;          // [E, d_model]
    const half_t* router_b;          // [E] or null
    const half_t* const* tables;     // device array [4][E]: W1[e] ([d_ff, d_model]), b1[e] or null, W2[e] ([d_model, d_ff]), b2[e] or null
    half_t* y;                       // [d_model]
    half_t* router_logits;           // [E] or null
    int* expert;                     // [1] or null
    unsigned long long* hx;          // [2][blocks][kMoeEntryWords]
    unsigned int* g_counter;         // [blocks][kMoeCounterStride]: every block's copy of the launch count in word 0 of its line
    unsigned int* abort_flag;        // device word: non-zero from the first wait that gave up until the host clears it
    unsigned int* abort_host;        // the same event for the host to see
    int d_model, d_ff, E, act, scale_by_prob;
    int wpb;                         // 16-byte words of hidden values per producing block
    int rpb2;                        // rows of W2 per block
    unsigned int spin_limit;
    int alone;                       // non-zero: every block computes all hidden values itself, nothing is exchanged
    int count_stride;                // 0: one launch count, advanced by block 0; kMoeCounterStride: one per block
};

// What the kernel's first instructions need comes as plain arguments in front of the struct: those arrive in scalar
// registers with the wavefront (kernel-argument preload) instead of through a load at its start.
__global__ __launch_bounds__(kMoeThreads) void moe_ffn_step_f16_kernel(const half_t* x_, const half_t* router_w_, const half_t* router_b_,
                                                                       const half_t* const* tables_, int d_model_, int d_ff_, int E_, int act_,
                                                                       MoeStepArgs p)
{
    p.x = x_;
    p.router_w = router_w_;
    p.router_b = router_b_;
    p.tables = tables_;
    p.d_model = d_model_;
    p.d_ff = d_ff_;
    p.E = E_;
    p.act = act_;
    __shared__ __align__(16) half_t hidden[kMoeMaxFf];
    __shared__ float logit_s[kMoeMaxExperts];
    __shared__ const half_t* table_s[4][kMoeMaxExperts];
    __shared__ __align__(16) unsigned short mine[8 * kMoeMaxWordsPerBlock];  // this block's hidden values (bits)
    __shared__ int someone_gave_up;
    __shared__ int block_poisoned;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = blockIdx.x, nb = gridDim.x;
    const int nx = p.d_model >> 3, nf = p.d_ff >> 3;  // 16-byte pieces of a W1 / W2 row; nf is also the number of hidden words
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;

    if (tid == 0) {
        someone_gave_up = 0;
        block_poisoned = 0;
    }
    // the experts' pointers, while the router's rows travel
    for (int i = tid; i < 4 * p.E; i += kMoeThreads) table_s[i / p.E][i % p.E] = p.tables[i];

    // ---- the token, then the router: every block computes all E logits ----
    half8_t xr[kMoeXC];
    const half8_t* x8 = reinterpret_cast<const half8_t*>(p.x);
#pragma unroll
    for (int k = 0; k < kMoeXC; ++k) xr[k] = (lane + 64 * k < nx) ? x8[lane + 64 * k] : zero8;
    // (two experts per wavefront and pass: all their loads are in flight together, one round trip for E <= 16)
    for (int e0 = wave; e0 < p.E; e0 += 2 * kMoeWaves) {
        const int e1 = e0 + kMoeWaves;
        const half8_t* w8a = reinterpret_cast<const half8_t*>(p.router_w) + (long)e0 * nx;
        const half8_t* w8b = reinterpret_cast<const half8_t*>(p.router_w) + (long)(e1 < p.E ? e1 : e0) * nx;
        half8_t ra[kMoeXC], rb[kMoeXC];
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k) {
            if (64 * k >= nx) break;  // (uniform) pieces past the row for every lane
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

    // One row of W1[e] times the token, bias and activation, as the bits `hidden` holds; a NaN in its canonical form.
    auto hidden_bits = [&](float a, int r) {
        if (b1) a += (float)b1[r];
        if (p.act == 1) a = relu_f32(a);
        unsigned short bits = __builtin_bit_cast(unsigned short, (half_t)a);
        if (a != a) bits = 0x7e00u;
        return bits;
    };
    // This wavefront's row of W2[e]: asked for here, consumed at the end.
    half8_t w2r[kMoeFC];
    const int r2 = b * p.rpb2 + wave;
    const bool has_row2 = wave < p.rpb2 && r2 < p.d_model;
    auto ask_for_w2 = [&]() {
        const half8_t* src = w2 + (long)min(r2, p.d_model - 1) * nf;  // (a row this wavefront does not own is loaded and dropped)
#pragma unroll
        for (int k = 0; k < kMoeFC; ++k) {
            if (64 * k >= nf) break;  // (uniform) pieces past the row for every lane
            w2r[k] = load_weight<true>(src + min(lane + 64 * k, nf - 1));
        }
    };

    // The launch count (which set of slots this launch uses) and the abort word are device-scope loads, which take longer
    // than the cached ones above and would hold those up if they stood in front of them (a wavefront's loads return in
    // order).  Asked for here, they travel with the rows of W1 and are needed when the block publishes.
        const unsigned int g = __hip_atomic_load(p.g_counter + p.count_stride * b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned int poisoned = __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // ---- hidden = act(W1[e] . x + b1[e]): this block's words (asked for whether or not they will be published) ----
    const int row0 = 8 * p.wpb * b + wave * p.wpb;  // this wavefront's first row
    half8_t w1r[kMoeMaxWordsPerBlock][kMoeXC];
#pragma unroll
    for (int s = 0; s < kMoeMaxWordsPerBlock; ++s) {
        const int r = min(row0 + min(s, p.wpb - 1), p.d_ff - 1);
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k) {
            if (64 * k >= nx) break;
            w1r[s][k] = load_weight<true>(w1 + (long)r * nx + min(lane + 64 * k, nx - 1));
        }
    }
#pragma unroll
    for (int s = 0; s < kMoeMaxWordsPerBlock; ++s) {
        const int r = row0 + s;
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kMoeXC; ++k)
            if (lane + 64 * k < nx) a = dot8(w1r[s][k], xr[k], a);
        a = wave_sum(a);
        if (lane == 0 && s < p.wpb) mine[wave * p.wpb + s] = r < p.d_ff ? hidden_bits(a, r) : (unsigned short)0;
    }
    // Whether the abort word is up is decided for the block as a whole, through LDS: wavefronts look at it at slightly
    // different times and can see different values when it is raised while the launch starts; they would then disagree
    // about the barriers that follow.  (The flags were set to 0 in front of the barrier behind the router.)
    if (poisoned != 0u) block_poisoned = 1;
    __syncthreads();
    const bool alone = p.alone != 0 || block_poisoned != 0;
    const unsigned int set = g & 1u;
    if (!alone) {
        if (tid < p.wpb && b * p.wpb + tid < nf) {
            const unsigned long long* src = reinterpret_cast<const unsigned long long*>(&mine[8 * tid]);
            store16_device_scope(p.hx + ((long)set * nb + b) * kMoeEntryWords + 2 * tid, src[0], src[1]);
        }
        ask_for_w2();
        // ---- everybody's hidden values: thread t takes word t ----
        if (tid < nf) {
            const unsigned long long* slot = p.hx + ((long)set * nb + tid / p.wpb) * kMoeEntryWords + 2 * (tid % p.wpb);
            unsigned long long lo = kMoeEmpty, hi = kMoeEmpty;
            unsigned int spins = 0;
            unsigned long long t_first = 0ull;
            bool gave_up = false;
            while (true) {
                load16_device_scope(slot, lo, hi);
                if (lo != kMoeEmpty && hi != kMoeEmpty) break;
                if (spins > 0u && (spins & 255u) == 0u) {
                    if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                    if (wait_clock_expired(spins, t_first)) spins = 0xffffffffu;  // gives up below
                }
                if (spins >= p.spin_limit) {  // (with a limit of 0 a lane whose first look failed gives up without another)
                    __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    gave_up = true;
                }
                if (gave_up) break;
                if (spins != 0xffffffffu) ++spins;
            }
            if (gave_up) someone_gave_up = 1;
            typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
            const u64x2 v = {lo, hi};
            *reinterpret_cast<u64x2*>(&hidden[8 * tid]) = v;
        }
        __syncthreads();
    } else {
        ask_for_w2();
        __syncthreads();
    }
    if (alone || someone_gave_up) {
        // ---- self-sufficient: every hidden value from W1[e], by this block alone ----
        for (int r = wave; r < p.d_ff; r += kMoeWaves) {
            float a = 0.0f;
#pragma unroll
            for (int k = 0; k < kMoeXC; ++k)
                if (lane + 64 * k < nx) a = dot8(w1[(long)r * nx + lane + 64 * k], xr[k], a);
            a = wave_sum(a);
            if (lane == 0) hidden[r] = __builtin_bit_cast(half_t, hidden_bits(a, r));
        }
        __syncthreads();
    }

    // ---- y = W2[e] . hidden + b2[e] ----
    {
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kMoeFC; ++k) {
            const int c = lane + 64 * k;
            if (c < nf) a = dot8(w2r[k], *reinterpret_cast<const half8_t*>(&hidden[c * 8]), a);
        }
        a = wave_sum(a);
        if (lane == 0 && has_row2) {
            if (b2) a += (float)b2[r2];
            p.y[r2] = (half_t)(a * scale);
        }
    }
    // this block's entry of the other set is empty for the next launch (nobody reads that set during this one)
    if (tid < 2 * kMoeMaxWordsPerBlock)
        __hip_atomic_store(p.hx + ((long)(set ^ 1u) * nb + b) * kMoeEntryWords + tid, kMoeEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0 && (b == 0 || p.count_stride != 0))
        __hip_atomic_store(p.g_counter + p.count_stride * b, g + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
