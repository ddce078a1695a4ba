// LSTM sequences with each recurrence confined to ONE XCD of the gfx950 part.
//
// lstm_seq_f16_kernel spreads a recurrence over every CU, so each step ends in an exchange of h between all eight
// XCDs, which has to go through the memory side (device scope): 1.4-1.8 us per step for 256 blocks, whatever the
// arithmetic.  The CUs of one XCD share an L2, and data that stays below it travels much faster: an all-to-all
// round among the 32 workgroups of one XCD takes 0.43 us when the polls are served by that L2 (measured; 0.85-1.5
// us with device-scope accesses between the same workgroups).  One XCD's registers hold one layer's W_hh
// (8.4 MB at H = 1024 against 16 MB of VGPRs), so here a recurrence is a GROUP of up to 32 workgroups on one XCD,
// 32 hidden units (one 64-byte entry) each, and different recurrences (the two directions of a layer; the layers of a
// stack, each fed by the one below through memory) run on different XCDs at the same time.
//
// Placement: the dispatcher deals the workgroups of a launch to the XCDs round-robin, workgroup b to XCD (b + o) % 8
// with a start o that belongs to the hardware queue and changes over a process's life (measured: 0 on a fresh queue, 6
// and 7 later).  So a workgroup asks the hardware where it is (XCC_ID): the group it joins is the one of that XCD, and
// its rank in the group is b / 8, which under any rotation gives every XCD ranks 0 .. grid / 8 - 1 exactly once.  A
// placement that is not a rotation leaves some rank of some group empty, and that group's first exchange times out
// (every wait is bounded); a rank that is taken twice is noticed at once through a claim word per (XCD, rank).
//
// Exchange inside a group: as in lstm_seq_f16_kernel every fp16 of an entry carries a flag in bit 14 (|h| <= 1 keeps
// it free) that tells the values of super-step g from those of g - 2 in the same slot, so every piece a reader gets
// validates itself.  That is what makes the cheap accesses safe: entries are written with plain stores (the per-CU
// cache is write-through, so they land in the XCD's L2) and read with non-temporal loads (a line read that way is
// dropped from the per-CU cache at once, so the next poll goes to the L2 again).  Nothing in the results depends on
// that cache behaviour: a stale piece fails its flag check and is polled again; only the time a poll takes does.
// Every wait is bounded (spin_limit polls, then the abort flag, as in lstm_seq_f16_kernel), and as there a workgroup one
// of whose waits gave up publishes nothing from then on and computes its units of the recurrence by itself at the end.
//
// A stack of unidirectional layers runs as a pipeline over the XCDs: layer k's recurrence (group R_k) on one XCD, and for
// k >= 1 a second group P_k on another XCD that holds W_ih of layer k and turns every h of layer k - 1 into layer k's
// input-projection row as soon as it exists.  R_{k-1} hands its h_t to P_k, and P_k its row to R_k, through buffers in
// memory with one slot per time step (device-scope stores and loads; a slot is written once per launch, so there is no
// flow control): the host fills them with all-ones bytes before the launch, a pattern that neither an fp16 h (a NaN is
// stored in its canonical form there) nor an fp32 sum can be, and a reader polls a slot until none of its elements is
// that pattern.  Those hand-overs cross XCDs and take about a microsecond, but they are not on the recurrences' critical
// path: P_k looks one step ahead while it multiplies, R_k starts a few steps late and from then on finds its rows
// waiting.  All groups then advance at the rate of one group, L layers in about the time of one.
//
// A workgroup has eight wavefronts; wavefront w owns hidden units 32 * rank + 4 * w .. + 3, one per row of 16 lanes:
// lane l keeps, of the four gate rows of unit l >> 4, the 8-wide column pieces 16 c + (l & 15), c = 0..7, in 128 registers
// for the whole sequence.  Per step: lanes 0..15 of every wavefront fetch one 16-byte piece of the group's entries into
// LDS, one barrier, four dot products of 64 columns per lane, a transposing reduction over the 16 lanes of a row that
// leaves gate g of the unit in lanes 4 g .. 4 g + 3 of the row, the gate arithmetic in the lanes of gate 0, and one
// 8-byte store of the wavefront's four new h values into the workgroup's entry.
#pragma once

#include <type_traits>

#include "lstm_kernels.h"
#include "lstm_solo.h"

namespace pimhip
{
static constexpr int kXcdCount = 8;                                   // XCDs of the part
static constexpr int kXcdMembers = 32;                                // workgroups of a group (CUs of an XCD)
static constexpr int kXcdWaves = 8;
static constexpr int kXcdThreads = 64 * kXcdWaves;
static constexpr int kXcdUnitsPerWave = 4;
static constexpr int kXcdUnitsPerBlock = kXcdWaves * kXcdUnitsPerWave;  // 32 units: one 64-byte entry
static constexpr int kXcdMaxH = 1024;                                 // 64 lanes x 16 columns = 32 members x 32 units
static constexpr int kXcdEntryWords = 16;                             // 32-bit words per entry
static constexpr int kXcdMaxChains = 4;
static constexpr int kXcdRegionWords = 2 * kXcdMembers * kXcdEntryWords;  // one chain's two slots

struct XcdChain {
    const half_t* w_hh;   // [4H, H]
    const float* xproj;   // [T, 4H] fp32 with biases: computed before the launch, or filled during it by the layer's P group
    const half_t* h0;     // [H]
    const half_t* c0;     // [H]
    half_t* y;            // row t at y + t * y_stride; null for an inner layer of a pipeline
    half_t* hn;           // [H]
    half_t* cn;           // [H]
    half_t* seq_out;      // [T][H], one slot per step, read by the P group of the layer above; null for the last layer
    int reverse;          // 1: t = T-1 .. 0
    int xproj_polled;     // 1: the rows of xproj are written during this launch (all-ones bytes = not yet)
    const half_t* res_in; // [T][H]: the layer's own input, added to its output (y and seq_out get h + in); null: no residual sum
    int res_polled;       // 1: res_in is the seq_out of the layer below, written during this launch (all-ones fp16 = not yet)
};

struct XcdProj {
    const half_t* w_ih;    // [4H, H] of the layer this group feeds
    const float* bsum;     // [4H] fp32 b_ih + b_hh
    const half_t* seq_in;  // [T][H]: the h of the layer below, slot t filled during this launch
    float* xp_out;         // [T][4H]: the xproj of the layer this group feeds
};

static constexpr int kXcdRoleProj = 9;  // role values: 0 none, 1 + k recurrence of chain k, kXcdRoleProj + j projection j
static constexpr unsigned long long kXcdWaitTicks = 100000000ull;  // one second of the 100 MHz clock
static constexpr int kXcdLag = 2;       // steps a recurrence fed by a P group lets that group get ahead before it starts

struct LstmXcdArgs {
    XcdChain chain[kXcdMaxChains];
    XcdProj proj[kXcdMaxChains - 1];  // proj[j] feeds chain[j + 1]
    int role[kXcdCount];       // what the group on the XCD with this hardware index runs
    unsigned int* claims;      // [kXcdCount][kXcdMembers]: the launch (a counter value of the plan) that last took (XCD, rank)
    unsigned int* hx;          // [kXcdMaxChains] regions of kXcdRegionWords; zero when the chain's counter is 2
    unsigned int* g_counter;   // [kXcdMaxChains] device words: super-steps a chain's region has seen so far, plus 2
    unsigned int* abort_flag;
    unsigned int* abort_host;
    long y_stride;
    int H;
    int T;
    unsigned int spin_limit;
};

// The barrier of a step: LDS traffic of this wavefront done, then s_barrier.  __syncthreads() would also wait for every
// global store and load the wavefront has in flight (its release semantics cover global memory), and some of those cross
// to another XCD and back; nothing that passes between the wavefronts of a workgroup here goes through global memory.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ void load16_nt(const void* p, unsigned long long& lo, unsigned long long& hi)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    lo = (unsigned long long)v[0] | ((unsigned long long)v[1] << 32);
    hi = (unsigned long long)v[2] | ((unsigned long long)v[3] << 32);
}

__device__ __forceinline__ void store8_plain(void* p, unsigned long long v)
{
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 w = {(unsigned int)v, (unsigned int)(v >> 32)};
    asm volatile("global_store_dwordx2 %0, %1, off" : : "v"(p), "v"(w) : "memory");
}

// The 16-bit values that lanes 0, 16, 32 and 48 hold, as one 64-bit word in lane 0 (other lanes: unspecified).
// v_permlane16_swap with both operands alike leaves lane 16's value beside lane 0's and lane 48's beside lane 32's;
// v_permlane32_swap then brings the upper pair down.
__device__ __forceinline__ unsigned long long pack_row_heads(unsigned int v16)
{
    unsigned int a = v16, b = v16;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    const unsigned int x = a | (b << 16);
    unsigned int c = x, d = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(c), "+v"(d));
    return (unsigned long long)c | ((unsigned long long)d << 32);
}

// acc[g], one partial sum per lane and gate, for the unit of this row of 16 lanes: returns, in every lane l, the sum over
// the 16 lanes of the row of gate ((l >> 2) & 3).  Each stage halves the number of values a lane holds and doubles the
// lanes they are summed over: mirrored lanes of the row (l ^ 15), mirrored lanes of half a row (l ^ 7), the quad.
__device__ __forceinline__ float row16_transpose_sum4(const float (&acc)[4], int lane)
{
    const bool b3 = lane & 8, b2 = lane & 4;
    float v2[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) v2[r] = (b3 ? acc[2 + r] : acc[r]) + dpp_mov_f32<kDppRowMirror>(b3 ? acc[r] : acc[2 + r]);
    float v = (b2 ? v2[1] : v2[0]) + dpp_mov_f32<kDppRowHalfMirror>(b2 ? v2[0] : v2[1]);
    v += dpp_mov_f32<kDppQuadXor1>(v);
    v += dpp_mov_f32<kDppQuadXor2>(v);
    return v;
}

// PIPE = false: groups that neither feed nor are fed across XCDs (a single layer, the two directions of one); everything
// that concerns P groups and the hand-overs is compiled out, which is worth 10 % of a step.
// RES = true: layers with a residual sum (out_t = h_t + in_t).  The sum is made where h leaves the workgroup: the wavefront
// that hands the previous step's 32 h values to the layer above adds the layer's own input of that step, which it asked
// for a step earlier, and stores y from there too (one step late; hn stays h).  Compiled in only for stacks that have such
// layers.
template <bool PIPE, bool RES>
__device__ __forceinline__ void lstm_xcd_body(const LstmXcdArgs& p)
{
    __shared__ __align__(16) half_t hbuf[2][kXcdMaxH];  // h of the previous step, double buffered by step parity
    __shared__ __align__(16) float xring[kXcdWaves][32][4][4];  // per wavefront: [step & 31][gate][unit] projection terms
    __shared__ __align__(16) unsigned long long hout[2][kXcdWaves];  // the workgroup's 32 new h values, for the layer above
    __shared__ unsigned short in_ring[2][kXcdUnitsPerBlock];        // RES: the layer's own input of the last two steps, for the sums
    // Raised by a wavefront one of whose waits gave up, always in front of a step's barrier, and read by all right behind
    // it: the workgroup then leaves the loop of steps together, publishes nothing more and computes its units by itself.
    __shared__ int block_gave_up;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int xcd = (int)hw_xcc_id();  // the XCD this workgroup runs on
    const int rank = blockIdx.x >> 3;
    if (xcd >= kXcdCount) {
        // An id outside 0..7: not the part this kernel is laid out for (the host checks the placement of a probe launch
        // before it chooses this kernel).  Reported like a rank taken twice; every other workgroup's waits are bounded.
        if (tid == 0) {
            __hip_atomic_store(p.abort_host + 1, (unsigned int)blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            __hip_atomic_store(p.abort_host + 2, (unsigned int)xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.abort_host, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        return;
    }
    const int role = p.role[xcd];
    const int H = p.H;
    const int T = p.T;
    const int members = (H + kXcdUnitsPerBlock - 1) / kXcdUnitsPerBlock;
    if (role == 0 || rank >= members) return;  // whole workgroups, before any barrier
    const bool is_proj = PIPE && role >= kXcdRoleProj;
    const int k = is_proj ? role - kXcdRoleProj + 1 : role - 1;  // the chain this group runs or feeds
    const XcdChain& ch = p.chain[k];
    const XcdProj& pj = p.proj[is_proj ? k - 1 : 0];

    bool gave_up = false;
    const unsigned int g_base = __builtin_amdgcn_readfirstlane(
        __hip_atomic_load(p.g_counter + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    // A wait of an earlier launch gave up and the host has not re-initialised the exchange since: nothing is exchanged in
    // this launch, every workgroup of a recurrence computes its units by itself.
    const bool poisoned = __builtin_amdgcn_readfirstlane(__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) != 0u;
    if (tid == 0) block_gave_up = poisoned ? 1 : 0;
    unsigned int* region = p.hx + (long)k * kXcdRegionWords;
    // This launch's mark on (XCD, rank): the counter value is new in every launch of the plan.  Found already there, two
    // workgroups of this launch share the rank, so another rank of the group is empty: not a rotation.
    unsigned int claimed_before = 0u;
    if (tid == 0)
        claimed_before = __hip_atomic_exchange(p.claims + xcd * kXcdMembers + rank, g_base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- weights into registers: gate g (LibTorch order i, f, g, o) of unit u0 + (lane >> 4), column pieces 16 c + (lane & 15)
    const int u0 = rank * kXcdUnitsPerBlock + wave * kXcdUnitsPerWave;
    const bool units_ok = u0 < H;  // H % 8 == 0: the four units of a wavefront are all inside or all outside
    const int cl = lane & 15;
    const half_t* wsrc = is_proj ? pj.w_ih : ch.w_hh;
    half8_t w[4][8];
    {
        half8_t zero;
#pragma unroll
        for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int col = (16 * c + cl) * 8;
                const bool ok = units_ok && col < H;
                const long off = ((long)g * H + (u0 + (lane >> 4))) * H + col;
                w[g][c] = ok ? *reinterpret_cast<const half8_t*>(wsrc + off) : zero;
            }
        }
        for (int i = tid; i < 2 * kXcdMaxH / 8; i += kXcdThreads) reinterpret_cast<half8_t*>(&hbuf[0][0])[i] = zero;
    }
    if (tid == 0 && claimed_before == g_base) {
        __hip_atomic_store(p.abort_host + 1, (unsigned int)blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(p.abort_host + 2, (unsigned int)xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p.abort_host, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    __syncthreads();

    // After the reduction lane l holds gate (l >> 2) & 3 of unit l >> 4.
    const int my_unit = u0 + (lane >> 4);
    const int my_gate = (lane >> 2) & 3;
    const int uc = units_ok ? my_unit : H - 1;
    // Lanes 0..31 of wavefronts 0..3 fetch piece 32 w + lane of an h vector: 8 fp16 = columns 8 q .. 8 q + 7.  (The other
    // wavefronts never poll: they are the ones that talk to other XCDs, and a wavefront's loads come back in order.)
    // A group that neither feeds nor is fed across XCDs spreads the polls over all eight wavefronts, 16 lanes each.
    const bool crosses = PIPE && (is_proj || ch.xproj_polled != 0 || ch.seq_out != nullptr || (RES && ch.res_in != nullptr));
    const int piece = crosses ? wave * 32 + lane : wave * 16 + lane;
    const bool polls = (crosses ? (wave < 4 && lane < 32) : lane < 16) && piece * 8 < H;

    // One bounded wait: `again` loads and tests; gives up like every wait of this kernel, after spin_limit polls, and
    // also after kXcdWaitTicks of the constant 100 MHz clock, however long a poll takes in the environment the kernel
    // finds itself in (a wait that succeeds does so within microseconds).
    auto bounded_wait = [&](auto again) __attribute__((always_inline)) {
        unsigned int spins = 0;
        unsigned long long t_first = 0ull;
        while (!again() && !gave_up) {
            ++spins;
            if ((spins & 255u) == 0u) {
                if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                const unsigned long long now = __builtin_amdgcn_s_memrealtime();
                if (spins == 256u) t_first = now;
                else if (now - t_first > kXcdWaitTicks) spins = 0xffffffffu;  // gives up below
            }
            if (spins >= p.spin_limit) {
                __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                gave_up = true;
            }
        }
    };
    // true if none of the four fp16 of the word is the all-ones pattern
    auto filled16 = [](unsigned long long v) {
        const unsigned long long x = ~v;  // an all-ones fp16 becomes zero
        return ((x & 0xffffull) != 0ull) && ((x & 0xffff0000ull) != 0ull) && ((x & 0xffff00000000ull) != 0ull) && ((x >> 48) != 0ull);
    };

    if (is_proj) {
        // ================= P group: xproj rows of layer k from the h of layer k - 1, step by step =================
        if (poisoned) return;  // (the recurrence it feeds makes its own rows then)
        const float bias = pj.bsum[(long)my_gate * H + uc];
        float* dst = pj.xp_out + (long)my_gate * H + uc;
        unsigned long long lo = 0ull, hi = 0ull;  // this lane's piece of the step ahead
        if (polls) {
            lo = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(pj.seq_in + piece * 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            hi = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(pj.seq_in + piece * 8) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        for (int t = 0; t < T; ++t) {
            half_t* hb = hbuf[t & 1];
            if (polls) {
                const unsigned long long* src = reinterpret_cast<const unsigned long long*>(pj.seq_in + (long)t * H + piece * 8);
                if (!(filled16(lo) && filled16(hi))) {
                    bounded_wait([&]() {
                        load16_device_scope(src, lo, hi);
                        return filled16(lo) && filled16(hi);
                    });
                }
                typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
                const u64x2 both = {lo, hi};
                *reinterpret_cast<half8_t*>(hb + piece * 8) = __builtin_bit_cast(half8_t, both);
            }
            if (gave_up) block_gave_up = 1;
            lds_barrier();
            const int dead = __builtin_amdgcn_readfirstlane(block_gave_up);  // (asked for with the reads of h, looked at where the row would leave)
            if (polls && t + 1 < T) {
                // the step ahead, in flight while this one is multiplied (tested at the top of the next iteration)
                const unsigned long long* nxt = reinterpret_cast<const unsigned long long*>(pj.seq_in + (long)(t + 1) * H + piece * 8);
                lo = __hip_atomic_load(nxt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                hi = __hip_atomic_load(nxt + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                if (c * 128 >= H) break;
                const half8_t hv = *reinterpret_cast<const half8_t*>(hb + (16 * c + cl) * 8);
#pragma unroll
                for (int g = 0; g < 4; ++g) acc[g] = dot8(w[g][c], hv, acc[g]);
            }
            const float v = row16_transpose_sum4(acc, lane) + bias;
            if (dead) return;  // rows made from a stale h must not reach the recurrence: it will make its own
            if (units_ok && (lane & 3) == 0)
                __hip_atomic_store(reinterpret_cast<unsigned int*>(dst + (long)t * 4 * H), __builtin_bit_cast(unsigned int, v), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }

    // ================= R group: the recurrence of chain k =================
    // Compiled once per combination of "its projection rows arrive during the launch" and "its h goes to a layer above":
    // a step is sensitive to every instruction on its path, and the plain combination should not carry the others'.
    auto recurrence = [&](auto polled_c, auto feeds_c, auto res_c) __attribute__((always_inline)) {
    constexpr bool polled = decltype(polled_c)::value;
    constexpr bool feeds = decltype(feeds_c)::value;
    constexpr bool res = decltype(res_c)::value;
    constexpr bool emits = feeds || res;  // the workgroup's h values leave through hout, one step late
    // Without a residual sum: lanes 0..3 of wavefront 4 hand step se's 32 h values to the layer above, 16 bytes each.
    auto emit = [&](int se) __attribute__((always_inline)) {
        const unsigned long long* src = &hout[se & 1][2 * lane];
        store16_device_scope(ch.seq_out + (long)se * H + rank * kXcdUnitsPerBlock + lane * 8, src[0], src[1]);
    };
    // With one: lanes 0..31 of wavefront 4, one value each: a handful of instructions per step (eight values in each of
    // four lanes took 0.1 us per step more).
    const int eu = rank * kXcdUnitsPerBlock + (lane & 31);  // the unit an emitting lane handles
    const bool sums = res && wave == 4 && lane < 32 && eu < H;
    // The input of step s is asked for right after that step's barrier, together with the projection rows two steps ahead
    // (it exists: the projection row made from it is in use), parked in LDS at the top of step s + 1 and added after
    // that step's barrier.  Every wavefront drains its loads once per step, so what matters is that the load leaves
    // early in the step: issued behind the sum of the step before, it cost 0.23 us per step.
    unsigned short in_ahead = 0xffffu;
    auto emit_sum = [&](int se) __attribute__((always_inline)) {
        unsigned short in_bits = in_ring[se & 1][lane & 31];
        if (ch.res_polled && in_bits == 0xffffu) {
            const unsigned short* rin = reinterpret_cast<const unsigned short*>(ch.res_in) + (long)se * H + eu;
            bounded_wait([&]() {
                in_bits = __hip_atomic_load(rin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return in_bits != 0xffffu;
            });
        }
        const unsigned short hbits = reinterpret_cast<const unsigned short*>(&hout[se & 1][0])[lane & 31];
        const float v = (float)__builtin_bit_cast(half_t, hbits) + (float)__builtin_bit_cast(half_t, in_bits);
        const unsigned short ob = (v == v) ? __builtin_bit_cast(unsigned short, (half_t)v) : (unsigned short)0x7e00u;
        if (ch.y) reinterpret_cast<unsigned short*>(ch.y)[(long)se * p.y_stride + eu] = ob;
        if (feeds)
            __hip_atomic_store(reinterpret_cast<unsigned short*>(ch.seq_out) + (long)se * H + eu, ob, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    float c_reg = (float)ch.c0[uc];
    const bool rev = ch.reverse != 0;

    // The input-projection term does not depend on h and must stay off the step's critical path: a wavefront's loads
    // return in order, so a poll issued behind a load that misses the L2 would wait for it.  Each wavefront keeps the
    // terms of its 16 rows for up to 32 steps in LDS.  Rows that exist before the launch are fetched 16 steps at a time,
    // ONE 16-byte load per lane every 16 steps (lane l: gate l & 3 of the wavefront's four units, adjacent in a row of
    // xproj, for step offset l >> 2).  Rows that a P group writes during the launch are fetched one element per lane two
    // steps ahead, right after the step's barrier so that the load travels while the step is computed, and tested when
    // they are used; the wavefronts that poll for h leave that to wavefronts 4..7, which fetch the elements of wavefront
    // w - 4 beside their own (a poll would have to wait for such a load to come back from the other XCD first).
    const int u0c = units_ok ? u0 : H - 4;
    auto fetch_xp = [&](int s0) {
        const int sx = min(s0 + (lane >> 2), T - 1);
        const int t = rev ? (T - 1 - sx) : sx;
        return *reinterpret_cast<const float4_t*>(ch.xproj + (long)t * 4 * H + (long)(lane & 3) * H + u0c);
    };
    auto deposit_xp = [&](int half, const float4_t v) {
        *reinterpret_cast<float4_t*>(&xring[wave][half * 16 + (lane >> 2)][lane & 3][0]) = v;
    };
    const unsigned int* xp_mine = reinterpret_cast<const unsigned int*>(ch.xproj + (long)my_gate * H + uc);  // + t * 4H
    const bool fetcher = wave >= 4;
    const unsigned int* xp_other =
        reinterpret_cast<const unsigned int*>(ch.xproj + (long)my_gate * H + min(max(u0 - 16, 0) + (lane >> 4), H - 1));  // wavefront w - 4's
    auto xp_bits_at = [&](int t) { return __hip_atomic_load(xp_mine + (long)t * 4 * H, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    auto wait_xp = [&](int t) {
        unsigned int bits = 0xffffffffu;
        bounded_wait([&]() {
            bits = xp_bits_at(t);
            return bits != 0xffffffffu;
        });
        return bits;
    };
    float4_t xp_next = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    unsigned int xp_ahead = 0xffffffffu, xp_ahead_other = 0xffffffffu;  // polled rows: the elements of step s + 2, loaded during step s
    if (!polled) {
        deposit_xp(0, fetch_xp(0));
        deposit_xp(1, fetch_xp(16));
    } else {
        // Let the P group get kXcdLag steps ahead, then take the first two rows.
        (void)wait_xp(min(kXcdLag, T - 1));
        reinterpret_cast<unsigned int&>(xring[wave][0][my_gate][lane >> 4]) = wait_xp(0);
        reinterpret_cast<unsigned int&>(xring[wave][1][my_gate][lane >> 4]) = wait_xp(min(1, T - 1));
    }

    for (int s = 0; s < T; ++s) {
        half_t* hb = hbuf[s & 1];
        if (!polled) {
            // steps s + 16 .. s + 31 are fetched when step s starts a half, and written over the half that has just been
            // used up one step later (this wavefront's poll in between has waited for them)
            if ((s & 15) == 0 && s > 0) xp_next = fetch_xp(s + 16);
            if ((s & 15) == 1 && s > 1) deposit_xp(((s >> 4) & 1) ^ 1, xp_next);
        } else if (fetcher && s >= 1 && s + 1 < T) {
            // loaded during step s - 1; read (by this wavefront and by wavefront w - 4) after the barrier of step s + 1
            reinterpret_cast<unsigned int&>(xring[wave][(s + 1) & 31][my_gate][lane >> 4]) = xp_ahead;
            reinterpret_cast<unsigned int&>(xring[wave - 4][(s + 1) & 31][my_gate][lane >> 4]) = xp_ahead_other;
        }
        if (sums && s > 0) in_ring[(s - 1) & 1][lane & 31] = in_ahead;  // read after this step's barrier
        // ---- 1. h of the previous step into LDS
        if (polls) {
            half8_t hv;
            if (s == 0) {
                hv = *reinterpret_cast<const half8_t*>(ch.h0 + piece * 8);
            } else {
                const unsigned int gp = g_base + (unsigned int)s - 1u;
                const unsigned long long want = ((gp >> 1) & 1u) ? 0x4000400040004000ull : 0ull;
                const unsigned char* src = reinterpret_cast<const unsigned char*>(region + (long)(gp & 1u) * kXcdMembers * kXcdEntryWords) + piece * 16;
                unsigned long long lo = 0ull, hi = 0ull;
                bounded_wait([&]() {
                    load16_nt(src, lo, hi);
                    return (lo & 0x4000400040004000ull) == want && (hi & 0x4000400040004000ull) == want;
                });
                lo &= 0xbfffbfffbfffbfffull;
                hi &= 0xbfffbfffbfffbfffull;
                typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
                const u64x2 both = {lo, hi};
                hv = __builtin_bit_cast(half8_t, both);
            }
            *reinterpret_cast<half8_t*>(hb + piece * 8) = hv;
        }
        if (gave_up) block_gave_up = 1;
        lds_barrier();
        // (the same value in every thread: it is written in front of barriers only.  Asked for here, with the reads of h,
        // and looked at where values would leave the workgroup: the step's arithmetic does not wait for it)
        const int dead = __builtin_amdgcn_readfirstlane(block_gave_up);
        if (polled && fetcher && s + 2 < T) {
            xp_ahead = xp_bits_at(s + 2);
            xp_ahead_other = __hip_atomic_load(xp_other + (long)(s + 2) * 4 * H, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The previous step's h of the whole workgroup (gathered in LDS before the barrier) goes to the layer above, from a
        // wavefront that does not poll.
        if (!res && feeds && s > 0 && wave == 4 && lane < 4 && rank * kXcdUnitsPerBlock + lane * 8 < H && !dead) emit(s - 1);
        if (sums) {
            in_ahead = __hip_atomic_load(reinterpret_cast<const unsigned short*>(ch.res_in) + (long)s * H + eu, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
            if (s > 0 && !dead) emit_sum(s - 1);
        }

        // ---- 2. the four gate rows of this row of lanes' unit
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c * 128 >= H) break;  // (uniform) column pieces 16 c .. 16 c + 15 lie past the hidden state
            const half8_t hv = *reinterpret_cast<const half8_t*>(hb + (16 * c + cl) * 8);
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(w[g][c], hv, acc[g]);
        }
        unsigned int xp_bits = reinterpret_cast<const unsigned int&>(xring[wave][s & 31][my_gate][lane >> 4]);
        if (polled && xp_bits == 0xffffffffu) xp_bits = wait_xp(s);  // the P group had not got there when it was fetched
        const float a = row16_transpose_sum4(acc, lane) + __builtin_bit_cast(float, xp_bits);
        const int t = rev ? (T - 1 - s) : s;

        // Every lane activates its own gate; a lane of gate 0 then finds gate f in its mirror within half the row (l ^ 7),
        // gate o in its mirror within the row (l ^ 15) and gate g in the mirror of that one (l ^ 8).  (The other lanes
        // combine the gates in another order; their c and h are never used.)
        const bool is_g = my_gate == 2;
        const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
        const float act = is_g ? 2.0f * sg - 1.0f : sg;
        const float g_i = act;
        const float g_f = dpp_mov_f32<kDppRowHalfMirror>(act);
        const float g_o = dpp_mov_f32<kDppRowMirror>(act);
        const float g_g = dpp_mov_f32<kDppRowMirror>(g_f);
        const float c_new = g_f * c_reg + g_i * g_g;
        const bool h_is_number = (c_new == c_new) && (g_o == g_o);
        const half_t h = (half_t)(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
        c_reg = c_new;

        // ---- 3. the wavefront's four h values: lanes 0, 16, 32, 48 hold them; lane 0 stores y and publishes
        const unsigned int hb16 = (unsigned int)__builtin_bit_cast(unsigned short, h);
        const unsigned int pb16 = h_is_number ? hb16 : 0u;       // a NaN cannot carry the flag: it is exchanged as 0, y keeps it
        const unsigned int sb16 = h_is_number ? hb16 : 0x7e00u;  // and goes to the layer above in its canonical form
        unsigned long long yw = 0ull, pw = 0ull, sw = 0ull;
        if constexpr (PIPE || RES) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                yw |= (unsigned long long)(unsigned int)__builtin_amdgcn_readlane((int)hb16, 16 * i) << (16 * i);
                pw |= (unsigned long long)(unsigned int)__builtin_amdgcn_readlane((int)pb16, 16 * i) << (16 * i);
                if (emits) sw |= (unsigned long long)(unsigned int)__builtin_amdgcn_readlane((int)sb16, 16 * i) << (16 * i);
            }
        } else {
            // Independent recurrences (a single layer, the two directions of a layer): gathered into lane 0 with two row swaps
            // each, 3 % of a step faster than eight v_readlane and the scalar shifts behind them.  (The kernel that runs
            // pipelines of layers keeps the scalar path: there the same change cost 1.5-5 %.)
            pw = pack_row_heads(pb16);
            yw = pack_row_heads(hb16);
        }
        // (a wavefront one of whose waits gave up after this step's barrier has made its h from stale values: it keeps them
        // to itself, and the group's other members stop at their next wait)
        const bool wave_gave_up = __builtin_amdgcn_ballot_w64(gave_up) != 0ull;
        if (lane == 0) {
            const unsigned int g = g_base + (unsigned int)s;
            const unsigned long long flag = ((g >> 1) & 1u) ? 0x4000400040004000ull : 0ull;
            // units past H publish zeros with the flag, so that every piece of a member's entry validates
            unsigned char* dst = reinterpret_cast<unsigned char*>(region + ((long)(g & 1u) * kXcdMembers + rank) * kXcdEntryWords) + wave * 8;
            if (!wave_gave_up && !dead) store8_plain(dst, (units_ok ? pw : 0ull) | flag);
            if (!res && units_ok && ch.y) *reinterpret_cast<unsigned long long*>(ch.y + (long)t * p.y_stride + u0) = yw;
            if (emits) hout[s & 1][wave] = sw;
        }
        if (s == T - 1 && units_ok && (lane & 15) == 0) {
            ch.hn[my_unit] = h;
            ch.cn[my_unit] = (half_t)c_new;
        }
        if (dead) break;  // (a step made on stale values: nothing of it has left the workgroup)
    }
    if (emits && sums) in_ring[(T - 1) & 1][lane & 31] = in_ahead;
    if (gave_up) block_gave_up = 1;
    lds_barrier();
    if (emits && !block_gave_up) {
        if (!res && wave == 4 && lane < 4 && rank * kXcdUnitsPerBlock + lane * 8 < H) emit(T - 1);
        if (sums) emit_sum(T - 1);
        if (gave_up) block_gave_up = 1;  // (the last sum's own wait)
    }
    lds_barrier();
    };
    const bool polled_rt = PIPE && ch.xproj_polled != 0;
    const bool feeds_rt = PIPE && ch.seq_out != nullptr;
    const bool res_rt = RES && ch.res_in != nullptr;
    if (poisoned) {
        // (nothing is exchanged)
    } else if (RES && res_rt) {
        if (!polled_rt && !feeds_rt) recurrence(std::false_type{}, std::false_type{}, std::true_type{});
        else if (!polled_rt) recurrence(std::false_type{}, std::true_type{}, std::true_type{});
        else if (!feeds_rt) recurrence(std::true_type{}, std::false_type{}, std::true_type{});
        else recurrence(std::true_type{}, std::true_type{}, std::true_type{});
    } else if (!PIPE || (!polled_rt && !feeds_rt)) recurrence(std::false_type{}, std::false_type{}, std::false_type{});
    else if (!polled_rt) recurrence(std::false_type{}, std::true_type{}, std::false_type{});
    else if (!feeds_rt) recurrence(std::true_type{}, std::false_type{}, std::false_type{});
    else recurrence(std::true_type{}, std::true_type{}, std::false_type{});
    if (block_gave_up) {
        // ---- self-sufficient: this workgroup's units of chain k, from the call's inputs, by this workgroup alone: the layers
        // below it in the launch are recomputed on the way (lstm_solo.h) ----
        SoloStack st;
        st.y_stride = p.y_stride;
        st.H = H;
        st.T = T;
        const int first = PIPE ? 0 : k;  // independent chains (the two directions of a layer) have their own projection rows
        st.n = k - first + 1;
        st.xproj = p.chain[first].xproj;
        st.res_in0 = RES ? p.chain[first].res_in : nullptr;
        st.reverse = ch.reverse;
#pragma unroll
        for (int j = 0; j < kXcdMaxChains; ++j) {
            if (first + j > k) break;
            const XcdChain& cj = p.chain[first + j];
            SoloLayer& ly = st.layer[j];
            ly.w_hh = cj.w_hh;
            ly.w_ih = j > 0 ? p.proj[first + j - 1].w_ih : nullptr;
            ly.bsum = j > 0 ? p.proj[first + j - 1].bsum : nullptr;
            ly.h0 = cj.h0;
            ly.c0 = cj.c0;
            ly.residual = (RES && cj.res_in != nullptr) ? 1 : 0;
            const bool mine = first + j == k;
            ly.y = mine ? cj.y : nullptr;
            ly.hn = cj.hn;
            ly.cn = cj.cn;
            ly.u_begin = mine ? min(rank * kXcdUnitsPerBlock, H) : 0;
            ly.u_end = mine ? min((rank + 1) * kXcdUnitsPerBlock, H) : 0;
        }
        lstm_solo_stack<kXcdThreads, PIPE ? kXcdMaxChains : 1, kXcdMaxH>(st);
        return;
    }
    // Rank 0 has finished its last step, for which (T >= 2) it needed what every member published one step earlier:
    // every member has read the counter by now.
    if (rank == 0 && tid == 0)
        __hip_atomic_store(p.g_counter + k, g_base + (unsigned int)T, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <bool PIPE>
__global__ __launch_bounds__(kXcdThreads) void lstm_xcd_f16_kernel(LstmXcdArgs p)
{
    lstm_xcd_body<PIPE, false>(p);
}

// The pipeline for stacks that have layers with a residual sum.
__global__ __launch_bounds__(kXcdThreads) void lstm_xcd_res_f16_kernel(LstmXcdArgs p)
{
    lstm_xcd_body<true, true>(p);
}

}  // namespace pimhip
