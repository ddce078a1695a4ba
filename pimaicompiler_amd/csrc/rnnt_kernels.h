// One launch for one (t, u) step of an RNN-transducer's greedy decoding loop (gfx950, batch 1, fp16 storage, fp32 sums):
//
//     prediction network   h_l, c_l = LSTM cell of layer l on (l == 0 ? x : h_{l-1}), (h_prev_l, c_prev_l)      l < L
//     joint network        hidden = relu(W1 . cat(f, g) + b1),  g = h_{L-1}          logits = W2 . hidden + b2
//
// The reference runs this per iteration of the loop as executeAtenLSTM1 with seq_len == 1
// (runtime/source/executor/op_executor/aten_ops_executor.cpp:2135-2307) followed by the joint network's products, the
// first of which RemoveCatForAddmm has split into two dependent addmm over f and g
// (compiler/source/frontend/optimizer/remove_cat_for_addmm.cpp:46-191): five operator calls, four kernels here when issued
// one by one.  The step is a chain of L + 2 dependent matrix-vector products over 4.7 MB of weights (RNNT: L = 2, H = 320,
// f 1024 wide, 512 joint units, 29 symbols); launches and the gaps between them cost more than the products.
//
// One launch, every workgroup resident, each with one role and its weights asked for at the start:
//   blocks [l * H/8, (l + 1) * H/8)      layer l: eight hidden units per block, one per wavefront (its four gate rows of
//                                         W_hh and W_ih); W_hh . h_prev is summed while the input travels
//   the next J/8 blocks                   eight rows of W1, one per wavefront; the columns over f are summed at once
//   the last ceil(V/8) blocks             eight rows of W2
// What one role makes the next needs whole: h of a layer, g, hidden.  It travels as 16-byte words of eight fp16 values,
// one word per producing block, in 128-byte entries of their own (hx[2][blocks][16 x 8 bytes]); a consumer's thread t polls
// word t of the vector it needs with one device-scope load per look.  An empty 8-byte half is all ones, which no four
// values written here can be (a NaN is written as 0x7e00).  The two sets of entries alternate by the launch count g; a
// launch empties its own entries of the other set, so nothing is cleared between launches and steps can be recorded into a
// HIP graph.  Every block keeps its own copy of the count (a device word it reads at its start and advances at its end; all
// copies are equal between launches): a single word advanced by one block could be read by a block that starts late after
// that block has already ended, and the late block would then look into the wrong set.
//
// With run_prediction == 0 (the loop emitted a blank: only the encoder frame changed) the layers' blocks do nothing and
// the joint network reads g = h_prev of the last layer where it lies.
//
// Sums run in one fixed order whoever computes them (per row: lane c takes 16-byte pieces c, c + 64, .. in ascending
// order, the hidden-state columns before the input columns, f before g; then one reduction tree), so a vector that a
// workgroup had to make for itself has the bits it would have had from its producers.
//
// A wait that gives up does not leave the result undefined.  Every wait is bounded (`spin_limit` polls, one second); a block
// in which a lane gave up computes the vector it waited for by itself from the step's inputs (the chain up to there by one
// workgroup: slower, tens of microseconds, but it needs nobody), with the same sums and therefore the same bits.  That is
// why hn / cn must not overlap h_prev / c_prev: the inputs of a step stay what they were until it has ended.  The block
// raises the plan's abort word, which stays up: every later launch starts self-sufficient until the host has refilled the
// entries and cleared the word.
#pragma once

#include "device_common.h"

namespace pimhip
{

constexpr int kRnntThreads = 512;
constexpr int kRnntWaves = kRnntThreads / 64;
constexpr int kRnntMaxLayers = 4;
constexpr int kRnntMaxBlocks = 256;
constexpr int kRnntMaxIn = 1024;                     // width of x
constexpr int kRnntMaxH = 1024;                      // hidden units per layer
constexpr int kRnntMaxEnc = 2048;                    // width of f
constexpr int kRnntMaxJoint = 2048;                  // joint units
constexpr int kRnntXC = kRnntMaxIn / 8 / 64;         // 16-byte pieces of a W_ih row per lane
constexpr int kRnntHC = kRnntMaxH / 8 / 64;          // ... of a W_hh row, or of the g columns of a W1 row
constexpr int kRnntFC = kRnntMaxEnc / 8 / 64;        // ... of the f columns of a W1 row
constexpr int kRnntJC = kRnntMaxJoint / 8 / 64;      // ... of a W2 row
constexpr int kRnntMaxVec = kRnntMaxJoint > kRnntMaxH ? kRnntMaxJoint : kRnntMaxH;
constexpr int kRnntEntryWords = 16;                  // 8-byte words per entry (128 bytes: no two entries in one line of the memory-side cache); the first two carry the values
constexpr unsigned long long kRnntEmpty = ~0ull;
constexpr int kRnntCounterStride = 16;               // 32-bit words between the blocks' copies of the launch count: a 64-byte line each
static_assert(kRnntMaxVec / 8 <= kRnntThreads, "thread t of a block polls word t");
static_assert(kRnntMaxIn >= kRnntMaxH, "layers above the first take h of the layer below as their input");

struct RnntLayer {
    const half_t* w_ih;   // [4H, in_w]
    const half_t* w_hh;   // [4H, H]
    const float* bsum;    // [4H] fp32 b_ih + b_hh, or null
    int in_w;
};

// What every role needs at once; these travel as plain kernel arguments in front of the struct (they arrive in scalar
// registers with the wavefront, kernel-argument preload, instead of through a load at its start).
struct RnntStepIo {
    const half_t* x;        // [layer[0].in_w]
    const half_t* h_prev;   // [L, H]
    const half_t* c_prev;   // [L, H]
    const half_t* f;        // [F]
    int L, H, J;
    int run_prediction;
};

struct RnntStepArgs {
    RnntLayer layer[kRnntMaxLayers];
    half_t* hn;             // [L, H]
    half_t* cn;             // [L, H]
    half_t* logits;         // [V]
    half_t* joint_hidden;   // [J] or null
    const half_t* w1;       // [J, F + H]
    const half_t* b1;       // [J] or null
    const half_t* w2;       // [V, J]
    const half_t* b2;       // [V] or null
    unsigned long long* hx; // [2][blocks][kRnntEntryWords]
    unsigned int* g_counter;    // [blocks][kRnntCounterStride]: launches the exchange has seen, every block's copy in a line of its own
    unsigned int* abort_flag;   // device word: non-zero from the first wait that gave up until the host clears it
    unsigned int* abort_host;   // the same event for the host to see
    int F, V;
    unsigned int spin_limit;
    int alone;              // non-zero: every block computes what it needs by itself, nothing is exchanged
};

// The barrier between the roles' phases: this wavefront's LDS traffic done, then s_barrier.  __syncthreads() would also wait
// until every global store of the wavefront has been acknowledged (h and c on their way to memory: about a microsecond),
// which nothing here depends on.
__device__ __forceinline__ void rnnt_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// An fp32 value rounded to fp16 in a step of its own.  Where the rounding is the only use of a multiply-add's result the
// compiler folds it into that instruction (v_fma_mixlo_f16), which rounds once instead of twice and differs in the last bit
// now and then; whoever computes a unit, in whatever surrounding code, has to get the same bits.
__device__ __forceinline__ half_t rnnt_round(float v)
{
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

// The bits a value travels as: a NaN in its canonical form (an all-ones half word means "empty").
__device__ __forceinline__ unsigned short rnnt_bits(float a)
{
    unsigned short bits = __builtin_bit_cast(unsigned short, rnnt_round(a));
    if (a != a) bits = 0x7e00u;
    return bits;
}

// acc += row[c] . vec[c] over the 16-byte pieces c = lane, lane + 64, .. < n, ascending (row, vec: any address space).
__device__ __forceinline__ float rnnt_row_dot(const half8_t* row, const half8_t* vec, int n, int lane, float acc)
{
    for (int c = lane; c < n; c += 64) acc = dot8(row[c], vec[c], acc);
    return acc;
}

template <int CTRL>
__device__ __forceinline__ float rnnt_dpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Sum over all lanes that share (lane & 3); every lane receives the total of its class.  Row rotations, then
// v_permlane16_swap / v_permlane32_swap (with a == b == v on entry, a + b is the pairwise sum in every lane): no trip
// through the LDS crossbar, which the generic shuffle takes.
__device__ __forceinline__ float rnnt_sum_mod4(float v)
{
    v += rnnt_dpp<0x124>(v);  // row_ror:4
    v += rnnt_dpp<0x128>(v);  // row_ror:8
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

// Sum over the 64 lanes; every lane returns the total.
__device__ __forceinline__ float rnnt_sum(float v)
{
    v += rnnt_dpp<kDppQuadXor1>(v);
    v += rnnt_dpp<kDppQuadXor2>(v);
    return rnnt_sum_mod4(v);
}

// One hidden unit's step from this lane's partial sums of its four gate rows (i, f, g, o).  The four sums are folded
// into one reduction (after two halving exchanges lane l holds gate l & 3 summed over its quad), lanes 0..3 of every quad
// activate one gate each (sigmoid and tanh(a) = 2 sigmoid(2a) - 1 on the hardware exp2 and reciprocal: absolute error
// below 1e-6), quad broadcasts hand the four gates to everybody.  Every lane returns the same c_new, h_new.  `bias` is
// the bias of gate lane & 3; c_prev the same in every lane.
__device__ __forceinline__ void rnnt_unit(const float acc[4], float bias, float c_prev, int lane, float& c_new, half_t& h_new)
{
    const bool b0 = lane & 1, b1 = lane & 2;
    const float s0 = acc[0], s1 = acc[2], s2 = acc[1], s3 = acc[3];  // slots {i, g, f, o}
    const float a0 = (b0 ? s2 : s0) + rnnt_dpp<kDppQuadXor1>(b0 ? s0 : s2);
    const float a1 = (b0 ? s3 : s1) + rnnt_dpp<kDppQuadXor1>(b0 ? s1 : s3);
    float a = (b1 ? a1 : a0) + rnnt_dpp<kDppQuadXor2>(b1 ? a0 : a1);
    a = rnnt_sum_mod4(a) + bias;
    const bool is_g = (lane & 3) == 2;
    const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
    const float act = is_g ? 2.0f * sg - 1.0f : sg;
    const float g_i = rnnt_dpp<0x00>(act);  // quad_perm broadcasts of lanes 0, 1, 2, 3 of the quad
    const float g_f = rnnt_dpp<0x55>(act);
    const float g_g = rnnt_dpp<0xAA>(act);
    const float g_o = rnnt_dpp<0xFF>(act);
    c_new = __builtin_fmaf(g_f, c_prev, g_i * g_g);
    h_new = rnnt_round(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
}

// The chain of the step up to `upto` by this workgroup alone: upto < L gives h of layer `upto`, upto == L the joint
// network's hidden vector.  Returns where the vector lies (one of the two LDS buffers).  Every thread calls it.
__device__ __forceinline__ const half_t* rnnt_solo(const RnntStepIo& io, const RnntStepArgs& p, int upto, half_t* buf0, half_t* buf1)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = io.H, nhp = H >> 3;
    half_t* cur = buf0;
    half_t* nxt = buf1;
    __syncthreads();
    if (io.run_prediction) {
        const int last = upto < io.L ? upto : io.L - 1;
        for (int l = 0; l <= last; ++l) {
            const RnntLayer ly = p.layer[l];
            const int nxp = ly.in_w >> 3;
            const half8_t* in = reinterpret_cast<const half8_t*>(l == 0 ? io.x : cur);
            const half8_t* hv = reinterpret_cast<const half8_t*>(io.h_prev + (long)l * H);
            for (int u = wave; u < H; u += kRnntWaves) {
                float a[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const long r = (long)g * H + u;
                    a[g] = rnnt_row_dot(reinterpret_cast<const half8_t*>(ly.w_hh + r * H), hv, nhp, lane, 0.0f);
                    a[g] = rnnt_row_dot(reinterpret_cast<const half8_t*>(ly.w_ih + r * ly.in_w), in, nxp, lane, a[g]);
                }
                float c_new;
                half_t h_new;
                rnnt_unit(a, ly.bsum ? ly.bsum[(long)(lane & 3) * H + u] : 0.0f, (float)io.c_prev[(long)l * H + u], lane, c_new, h_new);
                if (lane == 0) nxt[u] = __builtin_bit_cast(half_t, rnnt_bits((float)h_new));
            }
            __syncthreads();
            half_t* t = cur;
            cur = nxt;
            nxt = t;
        }
    }
    if (upto >= io.L) {
        const half8_t* gv = reinterpret_cast<const half8_t*>(io.run_prediction ? cur : io.h_prev + (long)(io.L - 1) * H);
        const half8_t* fv = reinterpret_cast<const half8_t*>(io.f);
        const int nfp = p.F >> 3;
        for (int r = wave; r < io.J; r += kRnntWaves) {
            const half8_t* row = reinterpret_cast<const half8_t*>(p.w1 + (long)r * (p.F + H));
            float a = rnnt_row_dot(row, fv, nfp, lane, 0.0f);
            a = rnnt_row_dot(row + nfp, gv, nhp, lane, a);
            a = rnnt_sum(a);
            if (lane == 0) {
                if (p.b1) a += (float)p.b1[r];
                nxt[r] = __builtin_bit_cast(half_t, rnnt_bits(relu_f32(a)));
            }
        }
        __syncthreads();
        cur = nxt;
    }
    return cur;
}

__global__ __launch_bounds__(kRnntThreads) void rnnt_step_f16_kernel(const half_t* x_, const half_t* h_prev_, const half_t* c_prev_,
                                                                    const half_t* f_, int L_, int H_, int J_, int run_prediction_,
                                                                    const RnntStepArgs p)
{
    const RnntStepIo io = {x_, h_prev_, c_prev_, f_, L_, H_, J_, run_prediction_};
    __shared__ __align__(16) half_t buf0[kRnntMaxVec];
    __shared__ __align__(16) half_t buf1[kRnntMaxVec];
    __shared__ __align__(16) unsigned short mine[8];  // this block's eight values (bits)
    __shared__ int someone_gave_up;
    __shared__ int block_poisoned;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb = gridDim.x;
    // Which role a workgroup takes goes by the XCD it runs on.  A launch reaches the eight XCDs one after another (the last
    // about a microsecond after the first: XCDs 0..3, then 7, 6, 5, 4, as timed on MI355X), and workgroup i runs on XCD i mod 8.
    // The first layer's blocks are the only ones that have all their inputs when they start, so everybody else waits for
    // them: they go to the XCDs that start first.  b is the workgroup's place in that order (those on XCDs 0..3 in front of
    // those on XCDs 4..7); roles and exchange entries go by b.  Where workgroups land otherwise, the step is as right as
    // ever and only slower.
    const int wg = blockIdx.x;
    const int n_front = (nb >> 3) * 4 + min(nb & 7, 4);
    const int b = (wg & 7) < 4 ? (wg >> 3) * 4 + (wg & 3) : n_front + (wg >> 3) * 4 + ((wg & 7) - 4);
    const int H = io.H, nhp = H >> 3, nwh = H >> 3, nwj = io.J >> 3;
    const int n_lstm = io.L * nwh;
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;
    if (tid == 0) {
        someone_gave_up = 0;
        block_poisoned = 0;
    }
    rnnt_barrier();

    unsigned int g = 0u, poisoned = 0u;
    // The launch count (which set of entries this launch uses) and the abort word are device-scope loads, which take
    // longer than cached ones and would hold those up if they stood in front of them (a wavefront's loads return in
    // order): every role asks for them behind its weights.
    auto ask_for_the_device_words = [&]() {
        g = __hip_atomic_load(p.g_counter + kRnntCounterStride * b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        poisoned = __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // Thread t takes word t of the vector that the blocks first .. first + nwords publish; the vector lands in buf0.
    // Returns whether a lane of this block gave up (uniform).  (One look in flight per word and block: several wavefronts
    // looking for the same words, staggered in time, make every look slower and the step 1 us longer.)
    auto gather = [&](int first, int nwords, unsigned int set) {
        if (tid < nwords) {
            const unsigned long long* slot = p.hx + ((long)set * nb + first + tid) * kRnntEntryWords;
            unsigned long long lo = kRnntEmpty, hi = kRnntEmpty;
            unsigned int spins = 0;
            unsigned long long t_first = 0ull;
            bool gave_up = false;
            while (true) {
                load16_device_scope(slot, lo, hi);
                if (lo != kRnntEmpty && hi != kRnntEmpty) break;
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
            *reinterpret_cast<u64x2*>(&buf0[8 * tid]) = v;
        }
        rnnt_barrier();
        return someone_gave_up != 0;
    };
    // The vector of level `level` (h of that layer; level L: the joint hidden vector) that blocks first .. publish.
    // Whether the abort word is up is decided for the block as a whole, through LDS: wavefronts look at it at slightly
    // different times and can see different values when it is raised while the launch starts; they would then disagree
    // about the barriers that follow.
    auto vector_of = [&](int level, int first, int nwords, unsigned int set) -> const half_t* {
        if (poisoned != 0u) block_poisoned = 1;
        rnnt_barrier();
        const bool alone = p.alone != 0 || block_poisoned != 0;
        if (!alone && !gather(first, nwords, set)) return buf0;
        return rnnt_solo(io, p, level, buf0, buf1);
    };
    auto publish = [&](unsigned int set) {
        rnnt_barrier();
        if (tid == 0 && !p.alone) {
            const unsigned long long* src = reinterpret_cast<const unsigned long long*>(mine);
            store16_device_scope(p.hx + ((long)set * nb + b) * kRnntEntryWords, src[0], src[1]);
        }
    };

    if (b < n_lstm && !io.run_prediction) {
        // a step of the joint network alone: nothing to compute here, but the entries still alternate
        ask_for_the_device_words();
    } else if (b < n_lstm) {
        // ---- a layer of the prediction network: unit u, gate rows u, H + u, 2H + u, 3H + u ----
        const int l = b / nwh, u = 8 * (b % nwh) + wave;
        const RnntLayer ly = p.layer[l];
        const int nxp = ly.in_w >> 3;
        half8_t whh[4][kRnntHC], wih[4][kRnntXC], hv[kRnntHC], xin[kRnntXC];
        const half8_t* h8 = reinterpret_cast<const half8_t*>(io.h_prev + (long)l * H);
#pragma unroll
        for (int k = 0; k < kRnntHC; ++k) hv[k] = (lane + 64 * k < nhp) ? h8[lane + 64 * k] : zero8;
#pragma unroll
        for (int gt = 0; gt < 4; ++gt) {
            const half8_t* row = reinterpret_cast<const half8_t*>(ly.w_hh + ((long)gt * H + u) * H);
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k) {
                if (64 * k >= nhp) break;  // (uniform) pieces past the row for every lane
                whh[gt][k] = row[min(lane + 64 * k, nhp - 1)];
            }
        }
#pragma unroll
        for (int gt = 0; gt < 4; ++gt) {
            const half8_t* row = reinterpret_cast<const half8_t*>(ly.w_ih + ((long)gt * H + u) * ly.in_w);
#pragma unroll
            for (int k = 0; k < kRnntXC; ++k) {
                if (64 * k >= nxp) break;
                wih[gt][k] = row[min(lane + 64 * k, nxp - 1)];
            }
        }
        if (l == 0) {
            const half8_t* x8 = reinterpret_cast<const half8_t*>(io.x);
#pragma unroll
            for (int k = 0; k < kRnntXC; ++k) xin[k] = (lane + 64 * k < nxp) ? x8[lane + 64 * k] : zero8;
        }
        const float bias = ly.bsum ? ly.bsum[(long)(lane & 3) * H + u] : 0.0f;
        const float c_prev = (float)io.c_prev[(long)l * H + u];
        ask_for_the_device_words();
        float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int gt = 0; gt < 4; ++gt) {
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k)
                if (lane + 64 * k < nhp) a[gt] = dot8(whh[gt][k], hv[k], a[gt]);
        }
        const unsigned int set = g & 1u;
        if (l > 0) {
            const half8_t* in = reinterpret_cast<const half8_t*>(vector_of(l - 1, (l - 1) * nwh, nwh, set));
#pragma unroll
            for (int k = 0; k < kRnntXC; ++k) xin[k] = (lane + 64 * k < nxp) ? in[lane + 64 * k] : zero8;
        }
#pragma unroll
        for (int gt = 0; gt < 4; ++gt) {
#pragma unroll
            for (int k = 0; k < kRnntXC; ++k)
                if (lane + 64 * k < nxp) a[gt] = dot8(wih[gt][k], xin[k], a[gt]);
        }
        float c_new;
        half_t h_new;
        rnnt_unit(a, bias, c_prev, lane, c_new, h_new);
        if (lane == 0) mine[wave] = rnnt_bits((float)h_new);
        publish(set);
        if (lane == 0) {  // (behind the word the next role waits for)
            p.hn[(long)l * H + u] = h_new;
            p.cn[(long)l * H + u] = rnnt_round(c_new);
        }
    } else if (b < n_lstm + nwj) {
        // ---- the joint network's first layer: row r of W1 over cat(f, g) ----
        const int r = 8 * (b - n_lstm) + wave;
        const int nfp = p.F >> 3;
        const half8_t* row = reinterpret_cast<const half8_t*>(p.w1 + (long)r * (p.F + H));
        half8_t wf[kRnntFC], wg[kRnntHC], fv[kRnntFC], gv[kRnntHC];
        const half8_t* f8 = reinterpret_cast<const half8_t*>(io.f);
#pragma unroll
        for (int k = 0; k < kRnntFC; ++k) fv[k] = (lane + 64 * k < nfp) ? f8[lane + 64 * k] : zero8;
#pragma unroll
        for (int k = 0; k < kRnntFC; ++k) {
            if (64 * k >= nfp) break;
            wf[k] = row[min(lane + 64 * k, nfp - 1)];
        }
#pragma unroll
        for (int k = 0; k < kRnntHC; ++k) {
            if (64 * k >= nhp) break;
            wg[k] = row[nfp + min(lane + 64 * k, nhp - 1)];
        }
        if (!io.run_prediction) {
            const half8_t* g8 = reinterpret_cast<const half8_t*>(io.h_prev + (long)(io.L - 1) * H);
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k) gv[k] = (lane + 64 * k < nhp) ? g8[lane + 64 * k] : zero8;
        }
        const float bias = (lane == 0 && p.b1) ? (float)p.b1[r] : 0.0f;
        ask_for_the_device_words();
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kRnntFC; ++k)
            if (lane + 64 * k < nfp) a = dot8(wf[k], fv[k], a);
        const unsigned int set = g & 1u;
        if (io.run_prediction) {
            const half8_t* in = reinterpret_cast<const half8_t*>(vector_of(io.L - 1, (io.L - 1) * nwh, nwh, set));
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k) gv[k] = (lane + 64 * k < nhp) ? in[lane + 64 * k] : zero8;
        }
#pragma unroll
        for (int k = 0; k < kRnntHC; ++k)
            if (lane + 64 * k < nhp) a = dot8(wg[k], gv[k], a);
        a = rnnt_sum(a);
        if (lane == 0) {
            const unsigned short bits = rnnt_bits(relu_f32(a + bias));
            mine[wave] = bits;
            if (p.joint_hidden) p.joint_hidden[r] = __builtin_bit_cast(half_t, bits);
        }
        publish(set);
    } else {
        // ---- the joint network's second layer: row v of W2 ----
        const int v = 8 * (b - n_lstm - nwj) + wave;
        const int njp = io.J >> 3;
        const half8_t* row = reinterpret_cast<const half8_t*>(p.w2 + (long)min(v, p.V - 1) * io.J);
        half8_t wv[kRnntJC];
#pragma unroll
        for (int k = 0; k < kRnntJC; ++k) {
            if (64 * k >= njp) break;
            wv[k] = row[min(lane + 64 * k, njp - 1)];
        }
        const float bias = (lane == 0 && p.b2 && v < p.V) ? (float)p.b2[v] : 0.0f;
        ask_for_the_device_words();
        const unsigned int set = g & 1u;
        const half8_t* in = reinterpret_cast<const half8_t*>(vector_of(io.L, n_lstm, nwj, set));
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < kRnntJC; ++k)
            if (lane + 64 * k < njp) a = dot8(wv[k], in[lane + 64 * k], a);
        a = rnnt_sum(a);
        if (lane == 0 && v < p.V) p.logits[v] = rnnt_round(a + bias);
    }
    // this block's entry of the other set is empty for the next launch (nobody reads that set during this one)
    const unsigned int set = g & 1u;
    if (tid < 2 && b < n_lstm + nwj)
        __hip_atomic_store(p.hx + ((long)(set ^ 1u) * nb + b) * kRnntEntryWords + tid, kRnntEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) __hip_atomic_store(p.g_counter + kRnntCounterStride * b, g + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
