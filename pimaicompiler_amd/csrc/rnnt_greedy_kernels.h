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
//     then, long before the next symbol is known; the joint blocks sum their rows over the NEXT frame while they wait.
//
// Exchange: 16-byte words in 128-byte entries as in the step kernel, in FOUR sets.  A producer's n-th word (n counts the
// prediction network's runs for the layers' blocks, steps for the joint and symbol blocks) goes to set n mod 4; at the start
// of round n it empties its entry of set (n + 1) mod 4, which holds round n - 3.  Everybody who reads that word has long
// done so: readers on the chain of a round cannot fall a round behind, and for the one exception, blocks of the prediction
// network, which nobody waits for in steps after a blank, the symbol blocks look at a count that every block keeps of the
// decisions it has taken in (`seen`) and do not publish step s before all have taken in step s - 2.
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

constexpr int kRnntGreedySets = 4;
constexpr int kRnntGreedyMaxVocab = 64;            // the argmax is one wavefront's ballot
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

__device__ __forceinline__ float rnnt_max(float v)
{
    v = fmaxf(v, rnnt_dpp<kDppQuadXor1>(v));
    v = fmaxf(v, rnnt_dpp<kDppQuadXor2>(v));
    v = fmaxf(v, rnnt_dpp<0x124>(v));
    v = fmaxf(v, rnnt_dpp<0x128>(v));
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = fmaxf(a, b);
    }
    {
        float a = v, b = v;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        v = fmaxf(a, b);
    }
    return v;
}

// torch.argmax over V <= 64 fp16 values: the first maximum, a NaN counting as the largest.  Every lane returns it.
__device__ __forceinline__ int rnnt_argmax(const half_t* lg, int V, int lane)
{
    const bool mine = lane < V;
    const float v = mine ? (float)lg[lane] : -__builtin_inff();
    const unsigned long long nan_mask = __ballot(mine && v != v);
    if (nan_mask) return __builtin_ctzll(nan_mask);
    const float m = rnnt_max(v);
    return __builtin_ctzll(__ballot(mine && v == m));
}

// The whole loop by one workgroup.  LDS: hs [L * H] (h of every layer), cs [L * H], tmp [max(H, J)], lg [64].
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
            if (lane == 0) tmp[r] = __builtin_bit_cast(half_t, rnnt_bits(fmaxf(a + (p.b1 ? (float)p.b1[r] : 0.0f), 0.0f)));
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
    __shared__ __align__(16) half_t buf0[kRnntMaxVec];            // the vector a role waits for
    __shared__ __align__(16) half_t own[kRnntMaxH];               // a layer's blocks: h of their layer; joint blocks: g
    __shared__ __align__(16) half_t lg[kRnntGreedyMaxVocab];      // the step's logits
    __shared__ __align__(16) half_t emb[kRnntGreedyEmbHalfs];     // first layer: the embedding rows and x0 behind them
    __shared__ __align__(16) unsigned short mine[8];
    __shared__ int someone_gave_up;
    __shared__ int i_decode_alone;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb = gridDim.x, b = blockIdx.x;
    const int H = p.H, nhp = H >> 3, nwh = H >> 3, nwj = p.J >> 3, nwv = (p.V + 7) >> 3;
    const int n_lstm = p.L * nwh;
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;

    // The solo decoder's arrays lie where the embedding rows lay (the team's loop is over by then).
    half_t* solo_hs = emb;
    half_t* solo_cs = emb + kRnntMaxLayers * kRnntMaxH;
    static_assert(2 * kRnntMaxLayers * kRnntMaxH <= kRnntGreedyEmbHalfs, "the solo decoder's state fits where the embedding rows lay");

    if (tid == 0) {
        someone_gave_up = (p.alone || __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) ? 1 : 0;
        i_decode_alone = 0;
    }
    __syncthreads();

    RnntGreedyState s = {0, 0, 0, -1, p.run_pred_first};
    int n_pred = 0, step = 0;

    // Thread t takes word t of the vector that blocks first .. first + nwords published in `set`; it lands in dst.
    // Returns whether the block has to leave the loop (uniform).
    auto gather = [&](int first, int nwords, int set, half_t* dst) {
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
                    if (wait_clock_expired(spins, t_first)) spins = 0xffffffffu;
                }
                if (spins >= p.spin_limit) {
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
            *reinterpret_cast<u64x2*>(&dst[8 * tid]) = v;
        }
        rnnt_barrier();
        return someone_gave_up != 0;
    };
    // This block's entry of the set after `round`'s becomes empty (it holds round - 3).
    auto empty_next = [&](int round) {
        if (tid < 2)
            __hip_atomic_store(p.hx + ((long)((round + 1) & 3) * nb + b) * kRnntEntryWords + tid, kRnntEmpty, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    };
    // mine[] goes out as this block's word of `round`.  The store that emptied this entry's successor, issued a round's work
    // ago, is acknowledged first: whoever sees this word and moves on to the next set finds it emptied.
    auto publish = [&](int round) {
        rnnt_barrier();
        if (tid == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const unsigned long long* src = reinterpret_cast<const unsigned long long*>(mine);
            store16_device_scope(p.hx + ((long)(round & 3) * nb + b) * kRnntEntryWords, src[0], src[1]);
        }
    };
    // The end of a step for every role: the logits arrive, everybody takes the same decision.  Returns false when the block
    // has to leave the loop.
    auto decide = [&]() {
        if (gather(n_lstm + nwj, nwv, step & 3, lg)) return false;
        if (tid == 0) __hip_atomic_store(p.seen + (long)kRnntSeenStride * b, (unsigned int)(step + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int k = rnnt_argmax(lg, p.V, lane);
        const int at = s.emitted;
        n_pred += s.run_pred;
        ++step;
        if (rnnt_greedy_advance(s, k, p.blank, p.max_per_frame) && b == 0 && tid == 0) p.symbols[at] = k;
        return true;
    };
    auto running = [&]() { return s.t < p.T && s.emitted < p.max_symbols; };

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
        if (l == 0) {
            // the rows the first layer will be asked for: embedding[0 .. emb_rows) and, behind them, x0
            if (p.emb_in_lds) {
                const half8_t* e8 = reinterpret_cast<const half8_t*>(p.embedding);
                half8_t* d8 = reinterpret_cast<half8_t*>(emb);
                const int n8 = p.emb_rows * nxp;
                for (int i = tid; i < n8; i += kRnntThreads) d8[i] = e8[i];
                const half8_t* x8 = reinterpret_cast<const half8_t*>(p.x0);
                for (int i = tid; i < nxp; i += kRnntThreads) d8[n8 + i] = x8[i];
            }
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
            rnnt_barrier();
            if (s.run_pred) {
                empty_next(n_pred);
                const half8_t* in;
                if (l == 0) {
                    const int row = s.label < 0 ? p.emb_rows : s.label;
                    in = p.emb_in_lds ? reinterpret_cast<const half8_t*>(emb) + (long)row * nxp
                                      : reinterpret_cast<const half8_t*>(s.label < 0 ? p.x0 : p.embedding + (long)s.label * ly.in_w);
                } else {
                    if (gather((l - 1) * nwh, nwh, n_pred & 3, buf0)) {
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
                if (lane == 0) mine[wave] = bits;
                publish(n_pred);
                // h of this layer, for W_hh at the next symbol
                if (gather(l * nwh, nwh, n_pred & 3, own)) {
                    ok = false;
                    break;
                }
                sum_hh();
            }
            ok = decide();
        }
        if (ok && lane == 0) {
            if (p.hn) p.hn[(long)l * H + u] = h_last;
            if (p.cn) p.cn[(long)l * H + u] = c_half;
        }
    } else if (someone_gave_up == 0 && b < n_lstm + nwj) {
        // ---- the joint network's first layer: row r of W1 over cat(f, g) ----
        const int r = 8 * (b - n_lstm) + wave;
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
        // this lane's part of the row's sum over frame `frame` (zero past the last frame: never used)
        auto sum_f = [&](int frame) {
            float a = 0.0f;
            if (frame < p.T) {
                const half8_t* f8 = reinterpret_cast<const half8_t*>(p.enc + (long)frame * p.F);
#pragma unroll
                for (int k = 0; k < kRnntFC; ++k)
                    if (lane + 64 * k < nfp) a = dot8(wf[k], f8[lane + 64 * k], a);
            }
            return a;
        };
        float af_cur = sum_f(0), af_nxt = sum_f(1);
        int t_cur = 0;
        bool ok = true;
        while (ok && running()) {
            rnnt_barrier();
            empty_next(step);
            if (s.t != t_cur) af_cur = af_nxt;
            if (s.run_pred) {
                if (gather((p.L - 1) * nwh, nwh, n_pred & 3, own)) {
                    ok = false;
                    break;
                }
            }
            const half8_t* gv = reinterpret_cast<const half8_t*>(own);
            float a = af_cur;
#pragma unroll
            for (int k = 0; k < kRnntHC; ++k)
                if (lane + 64 * k < nhp) a = dot8(wg[k], gv[lane + 64 * k], a);
            a = rnnt_sum(a);
            if (lane == 0) mine[wave] = rnnt_bits(fmaxf(a + bias, 0.0f));
            publish(step);
            // while the symbol blocks work: the row's sum over the frame after this one
            if (s.t != t_cur) {
                t_cur = s.t;
                af_nxt = sum_f(t_cur + 1);
            }
            ok = decide();
        }
    } else if (someone_gave_up == 0) {
        // ---- the joint network's second layer: row v of W2 ----
        const int v = 8 * (b - n_lstm - nwj) + wave;
        const int njp = p.J >> 3;
        const half8_t* row = reinterpret_cast<const half8_t*>(p.w2 + (long)min(v, p.V - 1) * p.J);
        half8_t wv[kRnntJC];
#pragma unroll
        for (int k = 0; k < kRnntJC; ++k) {
            if (64 * k >= njp) break;
            wv[k] = row[min(lane + 64 * k, njp - 1)];
        }
        const float bias = (lane == 0 && p.b2 && v < p.V) ? (float)p.b2[v] : 0.0f;
        bool ok = true;
        while (ok && running()) {
            rnnt_barrier();
            empty_next(step);
            // how far everybody has come (asked for now, looked at before this step's logits go out)
            unsigned int sv = 0u;
            if (tid < nb) sv = __hip_atomic_load(p.seen + (long)kRnntSeenStride * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (gather(n_lstm, nwj, step & 3, buf0)) {
                ok = false;
                break;
            }
            const half8_t* in = reinterpret_cast<const half8_t*>(buf0);
            float a = 0.0f;
#pragma unroll
            for (int k = 0; k < kRnntJC; ++k)
                if (lane + 64 * k < njp) a = dot8(wv[k], in[lane + 64 * k], a);
            a = rnnt_sum(a);
            if (lane == 0) mine[wave] = v < p.V ? rnnt_bits(a + bias) : (unsigned short)0xfc00u;  // (-inf past the last symbol)
            if (tid < nb) {
                // nobody is still to take in the decision of step - 2 (whose words the next step's start empties)
                unsigned int spins = 0;
                unsigned long long t_first = 0ull;
                while ((int)sv < step - 1) {
                    bool gave_up = false;
                    if (spins > 0u && (spins & 255u) == 0u) {
                        if (__hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) gave_up = true;
                        if (wait_clock_expired(spins, t_first)) spins = 0xffffffffu;
                    }
                    if (spins >= p.spin_limit) {
                        __hip_atomic_store(p.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                        gave_up = true;
                    }
                    if (gave_up) {
                        someone_gave_up = 1;
                        break;
                    }
                    if (spins != 0xffffffffu) ++spins;
                    sv = __hip_atomic_load(p.seen + (long)kRnntSeenStride * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            publish(step);  // (its barrier also carries someone_gave_up to everybody)
            if (someone_gave_up != 0) {
                ok = false;
                break;
            }
            ok = decide();
        }
    }

    // ---- the end: the team's result, or one workgroup decodes the utterance by itself ----
    __syncthreads();
    if (someone_gave_up != 0) {
        if (tid == 0) i_decode_alone = (p.alone || atomicCAS(p.solo_owner, 0u, 1u) == 0u) ? 1 : 0;
        __syncthreads();
        if (i_decode_alone) rnnt_greedy_solo(p, solo_hs, solo_cs, buf0, lg);
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
