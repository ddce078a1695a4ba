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
// Every wait is bounded (spin_limit polls, then the abort flag, as in lstm_seq_f16_kernel).
//
// A workgroup has eight wavefronts; wavefront w owns hidden units 32 * rank + 4 * w .. + 3, one per row of 16 lanes:
// lane l keeps, of the four gate rows of unit l >> 4, the 8-wide column pieces 16 c + (l & 15), c = 0..7, in 128 registers
// for the whole sequence.  Per step: lanes 0..15 of every wavefront fetch one 16-byte piece of the group's entries into
// LDS, one barrier, four dot products of 64 columns per lane, a transposing reduction over the 16 lanes of a row that
// leaves gate g of the unit in lanes 4 g .. 4 g + 3 of the row, the gate arithmetic in the lanes of gate 0, and one
// 8-byte store of the wavefront's four new h values into the workgroup's entry.
#pragma once

#include "lstm_kernels.h"

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
    const float* xproj;   // [T, 4H] fp32 with biases
    const half_t* h0;     // [H]
    const half_t* c0;     // [H]
    half_t* y;            // row t at y + t * y_stride
    half_t* hn;           // [H]
    half_t* cn;           // [H]
    int reverse;          // 1: t = T-1 .. 0
};

struct LstmXcdArgs {
    XcdChain chain[kXcdMaxChains];
    int role[kXcdCount];       // chain index + 1 of the group that runs on the XCD with this hardware index, 0: none
    unsigned int* claims;      // [kXcdCount][kXcdMembers]: the launch (its chain's counter value) that last took (XCD, rank)
    unsigned int* hx;          // [kXcdMaxChains] regions of kXcdRegionWords; zero when the chain's counter is 2
    unsigned int* g_counter;   // [kXcdMaxChains] device words: super-steps a chain's region has seen so far, plus 2
    unsigned int* abort_flag;
    unsigned int* abort_host;
    long y_stride;
    int H;
    int T;
    unsigned int spin_limit;
};

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

__global__ __launch_bounds__(kXcdThreads) void lstm_xcd_f16_kernel(LstmXcdArgs p)
{
    __shared__ __align__(16) half_t hbuf[2][kXcdMaxH];  // h of the previous step, double buffered by step parity
    __shared__ __align__(16) float xring[kXcdWaves][32][4][4];  // per wavefront: [step & 31][gate][unit] projection terms

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    // HW_REG_XCC_ID (hardware register 20), bits 3:0: the XCD this workgroup runs on.
    const int xcd = (int)(__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 7u);
    const int rank = blockIdx.x >> 3;
    const int role = p.role[xcd];
    const int H = p.H;
    const int T = p.T;
    const int members = (H + kXcdUnitsPerBlock - 1) / kXcdUnitsPerBlock;
    if (role == 0 || rank >= members) return;  // whole workgroups, before any barrier
    const int k = role - 1;
    const XcdChain& ch = p.chain[k];

    bool gave_up = false;
    const unsigned int g_base = __builtin_amdgcn_readfirstlane(
        __hip_atomic_load(p.g_counter + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
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
                w[g][c] = ok ? *reinterpret_cast<const half8_t*>(ch.w_hh + off) : zero;
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
    float c_reg = (float)ch.c0[uc];
    const bool rev = ch.reverse != 0;

    // The input-projection term does not depend on h and must stay off the step's critical path: a wavefront's loads
    // return in order, so a poll issued behind a load that misses the L2 would wait for it.  Each wavefront keeps the
    // terms of its 16 rows for 32 steps in LDS (two halves of 16 steps) and refills the half it has used up with ONE
    // 16-byte load per lane every 16 steps: lane l fetches gate l & 3 of the wavefront's four units (adjacent in a row of
    // xproj) for step offset l >> 2.
    const int u0c = units_ok ? u0 : H - 4;
    auto fetch_xp = [&](int s0) {
        const int sx = min(s0 + (lane >> 2), T - 1);
        const int t = rev ? (T - 1 - sx) : sx;
        return *reinterpret_cast<const float4_t*>(ch.xproj + (long)t * 4 * H + (long)(lane & 3) * H + u0c);
    };
    auto deposit_xp = [&](int half, const float4_t v) {
        *reinterpret_cast<float4_t*>(&xring[wave][half * 16 + (lane >> 2)][lane & 3][0]) = v;
    };
    deposit_xp(0, fetch_xp(0));
    deposit_xp(1, fetch_xp(16));
    float4_t xp_next = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // Lanes 0..15 of wavefront w fetch piece 16 w + lane of the group's entries: 8 fp16 = columns 8 q .. 8 q + 7 of h.
    const int piece = wave * 16 + lane;
    const bool polls = lane < 16 && piece * 8 < H;

    for (int s = 0; s < T; ++s) {
        half_t* hb = hbuf[s & 1];
        // Refill of the projection terms: steps s + 16 .. s + 31 are fetched when step s starts a half, and written over
        // the half that has just been used up one step later (this wavefront's poll in between has waited for them).
        if ((s & 15) == 0 && s > 0) xp_next = fetch_xp(s + 16);
        if ((s & 15) == 1 && s > 1) deposit_xp(((s >> 4) & 1) ^ 1, xp_next);
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
                unsigned int spins = 0;
                while (true) {
                    load16_nt(src, lo, hi);
                    if (((lo & 0x4000400040004000ull) == want && (hi & 0x4000400040004000ull) == want) || gave_up) break;
                    ++spins;
                    if ((spins & 255u) == 0u) {
                        if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                    }
                    if (spins >= p.spin_limit) {
                        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        gave_up = true;
                    }
                }
                lo &= 0xbfffbfffbfffbfffull;
                hi &= 0xbfffbfffbfffbfffull;
                typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
                const u64x2 both = {lo, hi};
                hv = __builtin_bit_cast(half8_t, both);
            }
            *reinterpret_cast<half8_t*>(hb + piece * 8) = hv;
        }
        __syncthreads();

        // ---- 2. the four gate rows of this row of lanes' unit
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c * 128 >= H) break;  // (uniform) column pieces 16 c .. 16 c + 15 lie past the hidden state
            const half8_t hv = *reinterpret_cast<const half8_t*>(hb + (16 * c + cl) * 8);
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[g] = dot8(w[g][c], hv, acc[g]);
        }
        const float a = row16_transpose_sum4(acc, lane) + xring[wave][s & 31][my_gate][lane >> 4];
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
        const unsigned int pb16 = h_is_number ? hb16 : 0u;  // a NaN cannot carry the flag: it is exchanged as 0, y keeps it
        unsigned long long yw = 0ull, pw = 0ull;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            yw |= (unsigned long long)(unsigned int)__builtin_amdgcn_readlane((int)hb16, 16 * i) << (16 * i);
            pw |= (unsigned long long)(unsigned int)__builtin_amdgcn_readlane((int)pb16, 16 * i) << (16 * i);
        }
        if (lane == 0) {
            const unsigned int g = g_base + (unsigned int)s;
            const unsigned long long flag = ((g >> 1) & 1u) ? 0x4000400040004000ull : 0ull;
            // units past H publish zeros with the flag, so that every piece of a member's entry validates
            unsigned char* dst = reinterpret_cast<unsigned char*>(region + ((long)(g & 1u) * kXcdMembers + rank) * kXcdEntryWords) + wave * 8;
            store8_plain(dst, (units_ok ? pw : 0ull) | flag);
            if (units_ok) *reinterpret_cast<unsigned long long*>(ch.y + (long)t * p.y_stride + u0) = yw;
        }
        if (s == T - 1 && units_ok && (lane & 15) == 0) {
            ch.hn[my_unit] = h;
            ch.cn[my_unit] = (half_t)c_new;
        }
    }
    // Rank 0 has finished its last step, for which (T >= 2) it needed what every member published one step earlier:
    // every member has read the counter by now.
    if (rank == 0 && tid == 0)
        __hip_atomic_store(p.g_counter + k, g_base + (unsigned int)T, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
