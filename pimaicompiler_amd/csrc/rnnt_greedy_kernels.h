// An RNN-transducer's whole greedy decoding loop over one utterance in one launch (gfx950, batch 1, fp16 storage, fp32 sums).
//
//     t = 0, last = start of sequence, state = (h0, c0); g, state = prediction(last, state)
//     while t < T and fewer than max_symbols emitted:
//         k = argmax(joint(enc[t], g))
//         if k == blank:  t += 1
//         else:           emit k; g, state = prediction(embedding[k], state); after max_per_frame symbols of one frame t += 1
//
// The reference interprets this loop operator by operator (prim::Loop,
// runtime/source/executor/op_executor/prim_ops_executor.cpp:820-875; per iteration executeAtenLSTM1 with seq_len == 1,
// aten_ops_executor.cpp:2135-2307, the joint network's products, aten_ops_executor.cpp:181-216, and executeAtenArgmax,
// aten_ops_executor.cpp:520-560, whose result the host reads before the next iteration): launches, gaps and a device-to-host
// round trip per step, far more than the 4.7 MB of weights cost.  rnnt_step_f16_kernel makes an iteration one launch; here
// the loop itself runs on the device:
//
//   * the same roles as the step kernel (blocks of eight hidden units per layer, of eight joint rows, of eight symbols),
//     but every workgroup stays for the whole utterance with its rows of the weights in registers: nothing is read again;
//   * the argmax is taken by every workgroup for itself from the logits that the symbol blocks publish, so the decision
//     travels with the hand-over that ends the step and every workgroup keeps the same loop state (t, symbols so far, ..);
//   * a layer's blocks also collect their own layer's h (what W_hh multiplies at the next symbol) and sum W_hh . h right
//     then, long before the next symbol is known;
//   * most steps of a real utterance are blanks, after which only the frame changes: the joint blocks do not wait for the
//     decision but publish the hidden vectors of the next steps as well, up to eight ahead, as if every decision in
//     between were a blank (the frames' columns are asked for a round earlier and their sums kept), and the symbol blocks
//     turn every hidden vector that arrives into logits, two per round.  When a symbol is emitted, g gets a new version
//     and what was computed ahead under the old one is simply never looked at.  A run of blanks then costs what the symbol
//     blocks' round costs, not two hand-overs per step.
//
// Exchange: 8-byte words of three fp16 values and a 16-bit tag, three words per producing block in a 128-byte entry of its
// own, written and read with device-scope accesses.  The tag says what the word belongs to: h of a layer carries the
// version of g (the count of the prediction network's runs), hidden vectors and logits carry the step and the version they
// were computed under; a word with another tag is "not there yet", so nothing is ever cleared and a stale word cannot be
// taken for a fresh one.  h lives in four sets by version, hidden vectors and logits in rings of sixteen by step.  A
// producer may overwrite what is sixteen steps old: for the joint blocks' entries that follows from the order of things
// (they run at most eight steps ahead of decisions that the symbol blocks have already published); the symbol blocks, whom
// a slow reader could fall sixteen steps behind (nobody waits for the layers' blocks during a run of blanks), look at a
// count that every block keeps of the decisions it has taken in (`seen`) before they reuse an entry.
//
// Waiting: a block looks at everything it waits for in one round ("pass"): the words of a vector by the first six
// wavefronts, the logits of the next four steps by the last two (of one step where there are more than 80 symbols).  What
// the block cannot go on without is polled until it is there, the rest is looked at once; one barrier ends the round, and
// a pass can take several decisions at once.
//
// Sums run in the order of the step kernel, c is rounded to fp16 after every run of the prediction network as it is when
// the state travels between launches: symbols and final state equal, bit for bit, those of a loop of pimhip_rnnt_step
// driven from the host.
//
// Every wait is bounded.  A workgroup whose wait gives up raises the abort word; every workgroup then leaves the loop at its
// next wait, and the first to claim `solo_owner` decodes the whole utterance again from its start by itself (slower, tens
// of microseconds per step, the same sums): a wait that gives up costs time, not the result.
#pragma once

#include "rnnt_kernels.h"

namespace pimhip
{

constexpr int kRnntGreedyVersions = 4;             // h of a layer: one entry per block and version of g, modulo this
constexpr int kRnntGreedyRing = 16;                // hidden vectors and logits: one entry per block and step, modulo this
constexpr int kRnntGreedyAhead = 8;                // steps the joint network runs ahead of the decisions
constexpr int kRnntGreedyLook = 4;                 // steps whose logits one pass looks at
static_assert(kRnntGreedyAhead < kRnntGreedyRing && (kRnntGreedyRing & (kRnntGreedyRing - 1)) == 0, "ring");
constexpr int kRnntGreedyMaxVocab = 512;           // symbols (the logits of the steps a pass looks at lie in LDS)
constexpr int kRnntGreedyWideVocab = 10;           // with more symbol blocks than this a pass looks at the logits of one step, not four
constexpr int kRnntGreedyEmbHalfs = 16384;         // embedding rows kept in LDS by the first layer's blocks (32 KB)
constexpr int kRnntSeenStride = 16;                // 32-bit words between the blocks' `seen` counts

struct RnntGreedyArgs {
    RnntLayer layer[kRnntMaxLayers];
    const half_t* w1;          // [J, F + H]
    const half_t* b1;          // [J] or null
    const half_t* w2;          // [V, J]
    const half_t* b2;          // [V] or null
    const half_t* enc;         // [T, F]
    const half_t* embedding;   // [emb_rows, in_w of layer 0]: row k is the prediction network's input after symbol k
    const half_t* x0;          // [in_w of layer 0]: its input before any symbol
    const half_t* h0;          // [L, H] or null (zeros)
    const half_t* c0;
    half_t* hn;                // [L, H] or null
    half_t* cn;
    int* symbols;              // [max_symbols]
    int* result;               // [8]: symbols emitted, frames consumed, steps taken, 1 if one workgroup decoded alone, whether the
                               // last symbol is still to be fed to the prediction network, the last symbol (-1: none), 0, 0
    unsigned long long* hx;    // [kRnntGreedySets][blocks][kRnntEntryWords], all ones at the start
    unsigned int* seen;        // [blocks][kRnntSeenStride], zero at the start
    unsigned int* solo_owner;  // zero at the start
    unsigned int* abort_flag;
    unsigned int* abort_host;
    int L, H, F, J, V, T;
    int emb_rows, emb_in_lds;
    int blank, max_symbols, max_per_frame;
    int run_pred_first;        // 0: the first step takes g = h0 of the last layer as it is (decoding goes on after a blank)
    unsigned int spin_limit;
    int alone;                 // the launch is one workgroup that decodes by itself
};

struct RnntGreedyState {
    int t, emitted, frame_syms, label, run_pred;
};

// What symbol k does to the loop; returns whether k was emitted.
__device__ __forceinline__ bool rnnt_greedy_advance(RnntGreedyState& s, int k, int blank, int max_per_frame)
{
    if (k == blank) {
        s.t += 1;
        s.frame_syms = 0;
        s.run_pred = 0;
        return false;
    }
    s.label = k;
    s.emitted += 1;
    s.frame_syms += 1;
    s.run_pred = 1;
    if (s.frame_syms >= max_per_frame) {
        s.t += 1;
        s.frame_syms = 0;
    }
    return true;
}

template <int CTRL>
__device__ __forceinline__ unsigned int rnnt_dpp_u32(unsigned int v)
{
    return (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}

// The maximum over the 64 lanes; every lane returns it.
__device__ __forceinline__ unsigned int rnnt_max_u32(unsigned int v)
{
    v = max(v, rnnt_dpp_u32<kDppQuadXor1>(v));
    v = max(v, rnnt_dpp_u32<kDppQuadXor2>(v));
    v = max(v, rnnt_dpp_u32<0x124>(v));
    v = max(v, rnnt_dpp_u32<0x128>(v));
    {
        unsigned int a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = max(a, b);
    }
    {
        unsigned int a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = max(a, b);
    }
    return v;
}

// torch.argmax over V fp16 values: the first maximum, a NaN counting as the largest.  Every lane returns it.  One integer
// maximum over keys: the value's bits made monotonic (-0 as +0, a NaN above everything) in front of the index counted from
// the top, so that of equal values the first wins.  A lane takes the values lane, lane + 64, ..
__device__ __forceinline__ int rnnt_argmax(const half_t* lg, int V, int lane)
{
    unsigned int key = 0u;
    for (int i = lane; i < V; i += 64) {
        unsigned int bits = __builtin_bit_cast(unsigned short, lg[i]);
        if (bits == 0x8000u) bits = 0u;
        unsigned int order = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
        if ((bits & 0x7fffu) > 0x7c00u) order = 0xffffu;
        key = max(key, (order << 16) | (unsigned int)(0xffff - i));
    }
    return 0xffff - (int)(rnnt_max_u32(key) & 0xffffu);
}

// The whole loop by one workgroup.  LDS: hs [L * H] (h of every layer), cs [L * H], tmp [max(H, J)], lg [V].
__device__ __forceinline__ void rnnt_greedy_solo(const RnntGreedyArgs& p, half_t* hs, half_t* cs, half_t* tmp, half_t* lg)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = p.H, nhp = H >> 3, nfp = p.F >> 3, njp = p.J >> 3;
    __syncthreads();
    for (int i = tid; i < p.L * H; i += kRnntThreads) {
        hs[i] = p.h0 ? p.h0[i] : (half_t)0.0f;
        cs[i] = p.c0 ? p.c0[i] : (half_t)0.0f;
    }
    __syncthreads();
    RnntGreedyState s = {0, 0, 0, -1, p.run_pred_first};
    int steps = 0;
    while (s.t < p.T && s.emitted < p.max_symbols) {
        if (s.run_pred) {
            const half_t* x = s.label < 0 ? p.x0 : p.embedding + (long)s.label * p.layer[0].in_w;
            for (int l = 0; l < p.L; ++l) {
                const RnntLayer ly = p.layer[l];
                const int nxp = ly.in_w >> 3;
                const half8_t* in = reinterpret_cast<const half8_t*>(l == 0 ? x : hs + (long)(l - 1) * H);
                const half8_t* hv = reinterpret_cast<const half8_t*>(hs + (long)l * H);
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
                    rnnt_unit(a, ly.bsum ? ly.bsum[(long)(lane & 3) * H + u] : 0.0f, (float)cs[(long)l * H + u], lane, c_new, h_new);
                    if (lane == 0) {
                        tmp[u] = __builtin_bit_cast(half_t, rnnt_bits((float)h_new));
                        cs[(long)l * H + u] = rnnt_round(c_new);
                    }
                }
                __syncthreads();
                for (int i = tid; i < H; i += kRnntThreads) hs[(long)l * H + i] = tmp[i];
                __syncthreads();
            }
        }
        const half8_t* fv = reinterpret_cast<const half8_t*>(p.enc + (long)s.t * p.F);
        const half8_t* gv = reinterpret_cast<const half8_t*>(hs + (long)(p.L - 1) * H);
        for (int r = wave; r < p.J; r += kRnntWaves) {
            const half8_t* row = reinterpret_cast<const half8_t*>(p.w1 + (long)r * (p.F + H));
            float a = rnnt_row_dot(row, fv, nfp, lane, 0.0f);
            a = rnnt_row_dot(row + nfp, gv, nhp, lane, a);
            a = rnnt_sum(a);
            if (lane == 0) tmp[r] = __builtin_bit_cast(half_t, rnnt_bits(relu_f32(a + (p.b1 ? (float)p.b1[r] : 0.0f))));
        }
        __syncthreads();
        for (int v = wave; v < p.V; v += kRnntWaves) {
            float a = rnnt_row_dot(reinterpret_cast<const half8_t*>(p.w2 + (long)v * p.J), reinterpret_cast<const half8_t*>(tmp), njp, lane, 0.0f);
            a = rnnt_sum(a);
            if (lane == 0) lg[v] = __builtin_bit_cast(half_t, rnnt_bits(a + (p.b2 ? (float)p.b2[v] : 0.0f)));
        }
        __syncthreads();
        const int k = rnnt_argmax(lg, p.V, lane);
        const int at = s.emitted;
        if (rnnt_greedy_advance(s, k, p.blank, p.max_per_frame) && tid == 0) p.symbols[at] = k;
        ++steps;
        __syncthreads();
    }
    for (int i = tid; i < p.L * H; i += kRnntThreads) {
        if (p.hn) p.hn[i] = hs[i];
        if (p.cn) p.cn[i] = cs[i];
    }
    if (tid == 0) {
        p.result[0] = s.emitted;
        p.result[1] = s.t;
        p.result[2] = steps;
        p.result[3] = 1;
        p.result[4] = s.run_pred;
        p.result[5] = s.label;
    }
}

__global__ __launch_bounds__(kRnntThreads) void rnnt_greedy_f16_kernel(const RnntGreedyArgs p)
{
    typedef unsigned long long u64;
    __shared__ __align__(16) half_t buf0[kRnntMaxVec];                              // the vector a role waits for
    __shared__ __align__(16) half_t own[kRnntMaxH];                                 // a layer's blocks: h of their layer; joint blocks: g
    __shared__ __align__(16) half_t lgs[2][kRnntGreedyLook][kRnntGreedyMaxVocab];   // the logits of the next steps, alternating per pass
    __shared__ __align__(16) half_t emb[kRnntGreedyEmbHalfs];                       // first layer: the embedding rows and x0 behind them
    __shared__ __align__(16) unsigned short mine[2][12];                            // this block's eight values, alternating per publish
    __shared__ int missing[3][3 + kRnntGreedyLook];                                 // per pass (rotating): something of the vector / of step j is not
                                                                                    // there yet; a wait has given up; something of a second vector is not there
    __shared__ int someone_gave_up;
    __shared__ int i_decode_alone;
    __shared__ int min_seen_lds;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb = gridDim.x, b = blockIdx.x;
    const int H = p.H, nhp = H >> 3, nwh = H >> 3, nwj = p.J >> 3, nwv = (p.V + 7) >> 3;
    const int n_lstm = p.L * nwh;

    // The solo decoder's arrays lie where the embedding rows lay (the team's loop is over by then).
    half_t* solo_hs = emb;
    half_t* solo_cs = emb + kRnntMaxLayers * kRnntMaxH;
    static_assert(2 * kRnntMaxLayers * kRnntMaxH <= kRnntGreedyEmbHalfs, "the solo decoder's state fits where the embedding rows lay");

    if (tid == 0) {
        someone_gave_up = (p.alone || __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) ? 1 : 0;
        i_decode_alone = 0;
    }
    if (tid < 3 * (3 + kRnntGreedyLook)) (&missing[0][0])[tid] = 0;
    if (tid < 24) (&mine[0][0])[tid] = 0;
    __syncthreads();

    RnntGreedyState s = {0, 0, 0, -1, p.run_pred_first};
    int n_pred = 0, step = 0;          // runs of the prediction network and steps so far
    unsigned int n_pass = 0, n_publish = 0, waited = 0;
    bool dead = false;                 // a wait of this block has given up (the same in every thread)
    unsigned long long t_first = 0ull;

    auto running = [&]() { return s.t < p.T && s.emitted < p.max_symbols; };
    // The version of g that the current step's joint network sees: runs of the prediction network started, less one.
    auto g_version = [&]() { return n_pred + s.run_pred - 1; };
    auto h_tag = [](int version) { return (unsigned int)(version & 0x7fff); };
    auto step_tag = [](int st, int version) { return (unsigned int)(((version & 0x7f) << 8) | (st & 0xff)); };
    auto h_entry = [&](int version, int block) { return p.hx + ((long)(version & (kRnntGreedyVersions - 1)) * n_lstm + block) * kRnntEntryWords; };
    auto hid_entry = [&](int st, int j) {
        return p.hx + ((long)kRnntGreedyVersions * n_lstm + (long)(st & (kRnntGreedyRing - 1)) * nwj + j) * kRnntEntryWords;
    };
    auto lg_entry = [&](int st, int j) {
        return p.hx + ((long)kRnntGreedyVersions * n_lstm + (long)kRnntGreedyRing * nwj + (long)(st & (kRnntGreedyRing - 1)) * nwv + j) * kRnntEntryWords;
    };

    // mine[] of this publish goes out as three 8-byte words of three values and the tag each.
    auto publish = [&](u64* entry, unsigned int tag) {
        rnnt_barrier();
        if (tid < 3) {
            const unsigned short* m = mine[n_publish & 1u] + 3 * tid;
            const u64 w = (u64)m[0] | ((u64)m[1] << 16) | ((u64)m[2] << 32) | ((u64)tag << 48);
            __hip_atomic_store(entry + tid, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        ++n_publish;
    };
    auto my_values = [&]() { return mine[n_publish & 1u]; };

    // One 8-byte word: looked at once, or (blocks) polled until it carries `tag` or the wait's limits are reached, in which
    // case the thread raises the abort words and this pass's "gave up" flag.  Returns whether the tag is there.
    auto fetch = [&](const u64* slot, unsigned int tag, bool blocks, int* miss, u64& w) {
        unsigned int spins = 0;
        unsigned long long first = 0ull;
        while (true) {
            w = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((unsigned int)(w >> 48) == tag) return true;
            if (!blocks) return false;
            bool give_up = false;
            if (spins > 0u && (spins & 255u) == 0u) {
                if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) give_up = true;
                if (wait_clock_expired(spins, first)) spins = 0xffffffffu;
            }
            if (spins >= p.spin_limit) {
                __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                give_up = true;
            }
            if (give_up) {
                miss[1 + kRnntGreedyLook] = 1;
                someone_gave_up = 1;
                return false;
            }
            if (spins != 0xffffffffu) ++spins;
        }
    };
    auto unpack = [&](u64 w, half_t* dst, int prod, int part) {
        unsigned short* d = reinterpret_cast<unsigned short*>(dst) + 8 * prod + 3 * part;
        d[0] = (unsigned short)w;
        d[1] = (unsigned short)(w >> 16);
        if (part < 2) d[2] = (unsigned short)(w >> 32);
    };
    // One round over everything this block waits for: the 8-byte words of a vector (n_vec producers from `vec`, tagged
    // vec_tag, values to vec_dst) by the first six wavefronts, and with want_steps the logits of the steps step .. step + 3
    // under the current version by the last two.  What the block cannot go on without is polled until it is there
    // (vec_blocks; step_blocks: the logits of `step`), the rest is looked at once.  Returns bit 0: the vector is complete;
    // bit 1 + j: the logits of step + j are.
    // A second vector (vec2, looked at once) is taken along where the first leaves threads free; bit 30 says it is complete.
    auto pass = [&](const u64* vec, int n_vec, unsigned int vec_tag, half_t* vec_dst, bool vec_blocks, bool want_steps, bool step_blocks,
                    const u64* vec2 = nullptr, int n_vec2 = 0, unsigned int vec2_tag = 0u, half_t* vec2_dst = nullptr) -> int {
        int* miss = missing[n_pass % 3u];
        u64 w;
        if (tid < 384) {
            for (int i = tid; i < 3 * (n_vec + n_vec2); i += 384) {
                const bool second = i >= 3 * n_vec;
                const int i2 = second ? i - 3 * n_vec : i;
                const int prod = i2 / 3, part = i2 - 3 * prod;
                if (!second) {
                    if (fetch(vec + (long)prod * kRnntEntryWords + part, vec_tag, vec_blocks, miss, w))
                        unpack(w, vec_dst, prod, part);
                    else
                        miss[0] = 1;
                } else {
                    if (fetch(vec2 + (long)prod * kRnntEntryWords + part, vec2_tag, false, miss, w))
                        unpack(w, vec2_dst, prod, part);
                    else
                        miss[2 + kRnntGreedyLook] = 1;
                }
            }
        } else if (want_steps) {
            // 32 threads per step for the logits of four steps, or (many symbols) all 128 for those of `step` alone
            const bool wide = nwv > kRnntGreedyWideVocab;
            const int per_step = wide ? 128 : 32;
            const int j = (tid - 384) / per_step, i0 = (tid - 384) - j * per_step;
            if (wide && tid - 384 < kRnntGreedyLook - 1) miss[2 + (tid - 384)] = 1;
            for (int i = i0; i < 3 * nwv; i += per_step) {
                const int prod = i / 3, part = i - 3 * prod;
                if (fetch(lg_entry(step + j, prod) + part, step_tag(step + j, g_version()), step_blocks && j == 0, miss, w))
                    unpack(w, lgs[n_pass & 1u][j], prod, part);
                else
                    miss[1 + j] = 1;
            }
        }
        rnnt_barrier();
        int r = (n_vec > 0 && miss[0] == 0) ? 1 : 0;
        if (want_steps) {
#pragma unroll
            for (int j = 0; j < kRnntGreedyLook; ++j)
                if (miss[1 + j] == 0) r |= 2 << j;
        }
        if (n_vec2 > 0 && miss[2 + kRnntGreedyLook] == 0) r |= 1 << 30;
        if (miss[1 + kRnntGreedyLook] != 0) dead = true;
        // the flags of the pass after the next are cleared now: their last readers passed this barrier, their next
        // writers come after the next one
        if (tid < 3 + kRnntGreedyLook) missing[(n_pass + 2u) % 3u][tid] = 0;
        ++n_pass;
        return r;
    };
    // After a pass that brought nothing: counts, and gives up when the limits are reached.  Everybody learns of it behind the
    // next pass's barrier, through that pass's flags (a word that thread 0 wrote now could be read by some threads of this
    // round and not by others).
    auto nothing_came = [&]() {
        if (tid == 0) {
            bool give_up = false;
            if (waited > 0u && (waited & 255u) == 0u) {
                if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) give_up = true;
                if (wait_clock_expired(waited, t_first)) waited = 0xffffffffu;
            }
            if (waited >= p.spin_limit) {
                __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                give_up = true;
            }
            if (give_up) {
                someone_gave_up = 1;
                missing[n_pass % 3u][1 + kRnntGreedyLook] = 1;
            }
            if (waited != 0xffffffffu) ++waited;
        }
    };
    auto something_came = [&]() {
        if (tid == 0) waited = 0u;
    };
    // Takes the decisions whose logits a pass found (bits 1.. of mask), in order, up to and including the first that emits a
    // symbol (what lies behind it was computed for a g that is no longer the current one).  Returns how many.
    auto take_decisions = [&](int mask) {
        int taken = 0;
#pragma unroll
        for (int j = 0; j < kRnntGreedyLook; ++j) {
            if (!(mask & (2 << j)) || !running()) break;
            const int k = rnnt_argmax(lgs[(n_pass - 1u) & 1u][j], p.V, lane);
            const int at = s.emitted;
            n_pred += s.run_pred;
            ++step;
            ++taken;
            if (rnnt_greedy_advance(s, k, p.blank, p.max_per_frame)) {
                if (b == 0 && tid == 0) p.symbols[at] = k;
                break;
            }
        }
        if (taken > 0 && tid == 0)
            __hip_atomic_store(p.seen + (long)kRnntSeenStride * b, (unsigned int)step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return taken;
    };
    // Waits for a vector.  Returns false when the block has to leave the loop.
    auto wait_for_vector = [&](const u64* vec, int n_vec, unsigned int tag, half_t* dst) {
        pass(vec, n_vec, tag, dst, true, false, false);
        return !dead;
    };
    // Waits until the decision of `step` can be taken, and takes those behind it too if their logits are there already.
    // Returns false when the block has to leave the loop.
    auto wait_for_decisions = [&]() {
        const int r = pass(nullptr, 0, 0u, nullptr, false, true, true);
        if (dead) return false;
        take_decisions(r);
        return true;
    };

    if (someone_gave_up == 0 && b < n_lstm) {
        // ---- a layer of the prediction network: unit u, gate rows u, H + u, 2H + u, 3H + u ----
        const int l = b / nwh, u = 8 * (b % nwh) + wave;
        const RnntLayer ly = p.layer[l];
        const int nxp = ly.in_w >> 3;
        half8_t whh[4][kRnntHC], wih[4][kRnntXC];
#pragma unroll
        for (int gt = 0; gt < 4; ++gt) {
            const half8_t* row = reinterpret_cast<const half8_t*>(ly.w_hh + ((long)gt * H + u) * H);
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k) {
                if (64 * k >= nhp) break;
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
        const float bias = ly.bsum ? ly.bsum[(long)(lane & 3) * H + u] : 0.0f;
        half_t c_half = p.c0 ? p.c0[(long)l * H + u] : (half_t)0.0f;
        half_t h_last = p.h0 ? p.h0[(long)l * H + u] : (half_t)0.0f;
        for (int i = tid; i < H; i += kRnntThreads) own[i] = p.h0 ? p.h0[(long)l * H + i] : (half_t)0.0f;
        if (l == 0 && p.emb_in_lds) {
            // the rows the first layer will be asked for: embedding[0 .. emb_rows) and, behind them, x0
            const half8_t* e8 = reinterpret_cast<const half8_t*>(p.embedding);
            half8_t* d8 = reinterpret_cast<half8_t*>(emb);
            const int n8 = p.emb_rows * nxp;
            for (int i = tid; i < n8; i += kRnntThreads) d8[i] = e8[i];
            const half8_t* x8 = reinterpret_cast<const half8_t*>(p.x0);
            if (x8)  // (null when the first step does not run the prediction network: never asked for then)
                for (int i = tid; i < nxp; i += kRnntThreads) d8[n8 + i] = x8[i];
        }
        __syncthreads();
        // W_hh . h of the layer, summed as soon as h is known
        float a_hh[4];
        auto sum_hh = [&]() {
            const half8_t* hv = reinterpret_cast<const half8_t*>(own);
#pragma unroll
            for (int gt = 0; gt < 4; ++gt) {
                a_hh[gt] = 0.0f;
#pragma unroll
                for (int k = 0; k < kRnntHC; ++k)
                    if (lane + 64 * k < nhp) a_hh[gt] = dot8(whh[gt][k], hv[lane + 64 * k], a_hh[gt]);
            }
        };
        sum_hh();
        bool ok = true;
        while (ok && running()) {
            if (s.run_pred) {
                const int version = n_pred;
                const half8_t* in;
                if (l == 0) {
                    const int row = s.label < 0 ? p.emb_rows : s.label;
                    in = p.emb_in_lds ? reinterpret_cast<const half8_t*>(emb) + (long)row * nxp
                                      : reinterpret_cast<const half8_t*>(s.label < 0 ? p.x0 : p.embedding + (long)s.label * ly.in_w);
                } else {
                    if (!wait_for_vector(h_entry(version, (l - 1) * nwh), nwh, h_tag(version), buf0)) {
                        ok = false;
                        break;
                    }
                    in = reinterpret_cast<const half8_t*>(buf0);
                }
                float a[4];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) {
                    a[gt] = a_hh[gt];
#pragma unroll
                    for (int k = 0; k < kRnntXC; ++k)
                        if (lane + 64 * k < nxp) a[gt] = dot8(wih[gt][k], in[lane + 64 * k], a[gt]);
                }
                float c_new;
                half_t h_new;
                rnnt_unit(a, bias, (float)c_half, lane, c_new, h_new);
                c_half = rnnt_round(c_new);
                const unsigned short bits = rnnt_bits((float)h_new);
                h_last = __builtin_bit_cast(half_t, bits);
                if (lane == 0) my_values()[wave] = bits;
                publish(h_entry(version, b), h_tag(version));
                // h of this layer, for W_hh at the next symbol
                if (!wait_for_vector(h_entry(version, l * nwh), nwh, h_tag(version), own)) {
                    ok = false;
                    break;
                }
                sum_hh();
            }
            ok = wait_for_decisions();
        }
        if (ok && lane == 0) {
            if (p.hn) p.hn[(long)l * H + u] = h_last;
            if (p.cn) p.cn[(long)l * H + u] = c_half;
        }
    } else if (someone_gave_up == 0 && b < n_lstm + nwj) {
        // ---- the joint network's first layer: row r of W1 over cat(f, g), for the current step and, while nothing else
        // is to do, for the steps behind it should they all be blanks ----
        const int jb = b - n_lstm, r = 8 * jb + wave;
        const int nfp = p.F >> 3;
        const half8_t* row = reinterpret_cast<const half8_t*>(p.w1 + (long)r * (p.F + H));
        half8_t wf[kRnntFC], wg[kRnntHC];
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
        const float bias = (lane == 0 && p.b1) ? (float)p.b1[r] : 0.0f;
        for (int i = tid; i < H; i += kRnntThreads) own[i] = p.h0 ? p.h0[(long)(p.L - 1) * H + i] : (half_t)0.0f;  // g before the first run
        __syncthreads();
        // this lane's part of the row's sum over a frame (nothing is read for a frame the utterance does not have)
        auto sum_f = [&](int frame) {
            float a = 0.0f;
            if (frame >= 0 && frame < p.T) {
                const half8_t* f8 = reinterpret_cast<const half8_t*>(p.enc + (long)frame * p.F);
#pragma unroll
                for (int k = 0; k < kRnntFC; ++k)
                    if (lane + 64 * k < nfp) a = dot8(wf[k], f8[lane + 64 * k], a);
            }
            return a;
        };
        // The sums over the frames around the current one are kept (per thread, in the LDS that the first layer's blocks
        // use for the embedding rows): frames [af_lo, af_hi) in slots frame mod 16.  A frame is summed once, ahead of its
        // turn, whatever the number of symbols it then emits.
        float* af_ring = reinterpret_cast<float*>(emb) + tid;
        static_assert(kRnntGreedyRing * kRnntThreads * sizeof(float) <= kRnntGreedyEmbHalfs * sizeof(half_t), "the ring of frame sums fits");
        int af_lo = 0, af_hi = 0;
        auto frame_keep = [&](int frame, float a) {
            if (frame != af_hi) af_lo = frame;
            af_hi = frame + 1;
            if (af_hi - af_lo > kRnntGreedyRing) af_lo = af_hi - kRnntGreedyRing;
            af_ring[(frame & (kRnntGreedyRing - 1)) * kRnntThreads] = a;
        };
        auto frame_sum = [&](int frame) {
            if (frame >= af_lo && frame < af_hi) return af_ring[(frame & (kRnntGreedyRing - 1)) * kRnntThreads];
            const float a = sum_f(frame);
            frame_keep(frame, a);
            return a;
        };
        int have_g = -1;          // the version of g in `own`
        int pub = 0;              // the next step to publish a hidden vector for
        frame_sum(0);
        bool ok = true;
        while (ok && running()) {
            const int version = g_version();
            if (version != have_g) {
                if (!wait_for_vector(h_entry(version, (p.L - 1) * nwh), nwh, h_tag(version), own)) {
                    ok = false;
                    break;
                }
                have_g = version;
                pub = step;
            }
            if (pub < step) pub = step;
            // the current step first, then up to kRnntGreedyAhead behind it: two per round while symbols come (the next g is
            // what matters then), more in a run of blanks, where running ahead is all there is to do
            const int per_round = s.run_pred ? 2 : 5;
            for (int i = 0; i < per_round; ++i) {
                const int frame = s.t + (pub - step);
                if (frame >= p.T || pub > step + kRnntGreedyAhead) break;
                const half8_t* gv = reinterpret_cast<const half8_t*>(own);
                float a = frame_sum(frame);
#pragma unroll
                for (int k = 0; k < kRnntHC; ++k)
                    if (lane + 64 * k < nhp) a = dot8(wg[k], gv[lane + 64 * k], a);
                a = rnnt_sum(a);
                if (lane == 0) my_values()[wave] = rnnt_bits(relu_f32(a + bias));
                publish(hid_entry(pub, jb), step_tag(pub, version));
                ++pub;
            }
            // The next frames the ring does not hold yet are asked for now and summed behind the wait for the decisions (their
            // columns travel while the symbol blocks work): up to four a round, as many as a round can publish.
            constexpr int kAsk = 4;
            static_assert(kRnntGreedyAhead + 1 + kAsk <= kRnntGreedyRing, "the ring holds what is asked for ahead");
            const int f_first = af_hi;
            int n_ask = 0;
            half8_t col[kAsk][kRnntFC];
#pragma unroll
            for (int q = 0; q < kAsk; ++q) {
                const int f = f_first + q;
                const bool ask = f < p.T && f <= s.t + kRnntGreedyAhead + kAsk;
                if (ask) n_ask = q + 1;
#pragma unroll
                for (int k = 0; k < kRnntFC; ++k)
                    col[q][k] = (ask && lane + 64 * k < nfp) ? reinterpret_cast<const half8_t*>(p.enc + (long)f * p.F)[lane + 64 * k] : wf[k];
            }
            ok = wait_for_decisions();
#pragma unroll
            for (int q = 0; q < kAsk; ++q) {
                if (q < n_ask) {
                    float a = 0.0f;
#pragma unroll
                    for (int k = 0; k < kRnntFC; ++k)
                        if (lane + 64 * k < nfp) a = dot8(wf[k], col[q][k], a);
                    frame_keep(f_first + q, a);
                }
            }
        }
    } else if (someone_gave_up == 0) {
        // ---- the joint network's second layer: row v of W2, for every hidden vector that arrives ----
        const int vb = b - n_lstm - nwj, v = 8 * vb + wave;
        const int njp = p.J >> 3;
        const half8_t* row = reinterpret_cast<const half8_t*>(p.w2 + (long)min(v, p.V - 1) * p.J);
        half8_t wv[kRnntJC];
#pragma unroll
        for (int k = 0; k < kRnntJC; ++k) {
            if (64 * k >= njp) break;
            wv[k] = row[min(lane + 64 * k, njp - 1)];
        }
        const float bias = (lane == 0 && p.b2 && v < p.V) ? (float)p.b2[v] : 0.0f;
        int pub = 0;              // the next step to publish logits for
        int have_version = g_version();
        int min_seen = 0;         // no block has taken in fewer decisions than this
        bool ok = true;
        while (ok && running()) {
            const int version = g_version();
            if (version != have_version) {
                have_version = version;
                pub = step;
            }
            if (pub < step) pub = step;
            const int frame = s.t + (pub - step);
            bool want = frame < p.T && pub <= step + kRnntGreedyAhead;
            if (want && pub - kRnntGreedyRing >= min_seen) {
                // The entry for step `pub` still holds step pub - ring: has everybody taken that decision in?
                if (tid == 0) min_seen_lds = 0x7fffffff;
                rnnt_barrier();
                if (tid < nb)
                    atomicMin(&min_seen_lds, (int)__hip_atomic_load(p.seen + (long)kRnntSeenStride * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                rnnt_barrier();
                min_seen = min_seen_lds;
                want = pub - kRnntGreedyRing < min_seen;
            }
            // the hidden vector of `step` itself is what everybody waits for (no decision can come before it): polled; one
            // of a later step is looked for once per round, between looks at the decisions
            // and the one behind it is taken along (to the LDS that the first layer's blocks use for the embedding rows)
            const bool want2 = want && frame + 1 < p.T && pub + 1 <= step + kRnntGreedyAhead && pub + 1 - kRnntGreedyRing < min_seen;
            const int r = pass(hid_entry(pub, 0), want ? nwj : 0, step_tag(pub, version), buf0, pub == step, true, false,
                               hid_entry(pub + 1, 0), want2 ? nwj : 0, step_tag(pub + 1, version), emb);
            if (dead) {
                ok = false;
                break;
            }
            if (r & 1) {
                const bool two = (r & (1 << 30)) != 0;
                const half8_t* in0 = reinterpret_cast<const half8_t*>(buf0);
                const half8_t* in1 = reinterpret_cast<const half8_t*>(emb);
                float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
                for (int k = 0; k < kRnntJC; ++k) {
                    if (lane + 64 * k < njp) {
                        a0 = dot8(wv[k], in0[lane + 64 * k], a0);
                        if (two) a1 = dot8(wv[k], in1[lane + 64 * k], a1);
                    }
                }
                a0 = rnnt_sum(a0);
                if (two) a1 = rnnt_sum(a1);
                if (lane == 0) {
                    mine[n_publish & 1u][wave] = v < p.V ? rnnt_bits(a0 + bias) : (unsigned short)0xfc00u;   // (-inf past the last symbol)
                    if (two) mine[(n_publish + 1u) & 1u][wave] = v < p.V ? rnnt_bits(a1 + bias) : (unsigned short)0xfc00u;
                }
                // both go out behind one barrier, from two wavefronts
                rnnt_barrier();
                const int which = tid >> 6, part = tid & 63;
                if (part < 3 && which < (two ? 2 : 1)) {
                    const unsigned short* m = mine[(n_publish + which) & 1u] + 3 * part;
                    const u64 w = (u64)m[0] | ((u64)m[1] << 16) | ((u64)m[2] << 32) | ((u64)step_tag(pub + which, version) << 48);
                    __hip_atomic_store(lg_entry(pub + which, vb) + part, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                n_publish += two ? 2u : 1u;
                pub += two ? 2 : 1;
            }
            const int taken = take_decisions(r);
            if ((r & 1) || taken > 0)
                something_came();
            else
                nothing_came();
        }
    }

    // ---- the end: the team's result, or one workgroup decodes the utterance by itself ----
    __syncthreads();
    if (someone_gave_up != 0) {
        if (tid == 0) i_decode_alone = (p.alone || atomicCAS(p.solo_owner, 0u, 1u) == 0u) ? 1 : 0;
        __syncthreads();
        if (i_decode_alone) rnnt_greedy_solo(p, solo_hs, solo_cs, buf0, &lgs[0][0][0]);
        return;
    }
    if (b == 0 && tid == 0) {
        p.result[0] = s.emitted;
        p.result[1] = s.t;
        p.result[2] = step;
        p.result[3] = 0;
        p.result[4] = s.run_pred;
        p.result[5] = s.label;
    }
}

}  // namespace pimhip
