// One launch for a whole decoder step of a GNMT-style LSTM stack (gfx950, batch 1, fp16 storage, fp32 gates).
//
// The reference runs such a step as a chain of separate operators, each a launch (or several) of its own
// (runtime/source/executor/op_executor/aten_ops_executor.cpp:2135-2307 executeAtenLSTM1 with seq_len == 1, :668-747
// executeAtenBmm for the attention context, :43-179 executeAtenAdd for the residual sums, :181-216 executeAtenAddmm for
// the classifier; runtime/source/executor/op_executor/miopen_ops_executor.cpp:170-228 for where the results land):
//
//     y_0 = lstm_0(x)                               ctx = att[1, S] . enc[S, H]
//     y_k = lstm_k(cat(in_k, ctx))   k >= 1         in_1 = y_0,  in_{k+1} = out_k
//     out_k = y_k + in_k  for the layers with a residual connection, else y_k
//     logits = W_c . out_last + b_c
//
// Each of these is a matrix-vector product of a few MB, so the chain is bound by launch ramps, not by bytes.  Here the
// step is ONE persistent launch.  Only W_ih[:, 0:H] . in_k depends on the layer before; W_hh . h_prev, the context
// columns W_ih[:, H:2H] . ctx and layer 0's input product do not, so every block streams those for all layers at once
// at the start, prefetches the dependent columns into registers, and the layers then hand their outputs over through
// the flagged exchange described below, one round per layer.  The classifier streams after the last round.
//
// Grid: NB = ceil(H / 4) blocks of 512 lanes, all resident at once (H <= 1024).  Block b owns hidden units 4b .. 4b+3 of
// every layer; two wavefronts share a unit and split the columns of every weight row between them (lane l of a
// wavefront holds one 16-byte piece of each row).  Accumulator slot v holds gate {i, g, f, o}[v], so that the
// transpose-sum leaves gate k in lane k (as in the sequence kernel).
//
// Exchange: hx[stage][NB] entries of 64 bytes, of which a block uses the first 8: its four fp16 outputs of layer
// `stage`.  |y| <= 1, so bit 14 of each fp16 carries a flag, the parity of the launch count g (a device word read at
// the start and advanced by block 0 at the end): a slot written by launch g - 1 cannot pass for launch g, and the buffer
// starts as zeros with g = 1.  A NaN (bit 14 set) travels as the otherwise unused pattern 0x3fff.  Every wait is bounded:
// after `spin_limit` polls a lane raises the abort flags, all lanes stop waiting, the kernel runs to its end with
// undefined results and the host reports a time-out.
#pragma once

#include "device_common.h"
#include "lstm_kernels.h"

namespace pimhip
{
static constexpr int kDecMaxLayers = 4;
static constexpr int kDecThreads = 512;
static constexpr int kDecUnits = 4;          // hidden units per block
static constexpr int kDecMaxH = 1024;        // 2 wavefronts x 64 lanes x 8 columns per row
static constexpr int kDecEntryWords = 16;    // 32-bit words between the entries of consecutive blocks (64 bytes)
static constexpr int kDecMaxCtxOuts = 4;
static constexpr unsigned short kDecNanCode = 0x3fffu;

struct DecoderLayerArgs {
    const half_t* w_ih;    // [4H, in_w]
    const half_t* w_hh;    // [4H, H]
    const float* bsum;     // [4H] fp32, b_ih + b_hh
    const half_t* h_prev;  // [H]
    const half_t* c_prev;  // [H]
    half_t* hn;            // [H]
    half_t* cn;            // [H]
    half_t* out;           // [H] or null: what the next layer sees (y, or y + in for a residual layer)
    int in_w;              // row length of w_ih: the width of x for a plain first layer, H without context, 2H with
    int takes_ctx;         // input = cat(in[H], ctx[H])
    int residual;          // out = y + in
};

struct DecoderStepArgs {
    DecoderLayerArgs layer[kDecMaxLayers];
    int n_layers;
    const half_t* x;       // input of layer 0 (without the context part), x_w elements
    int x_w;
    const half_t* ctx_in;  // [H] or null
    const half_t* att;     // [S]: ctx = att . enc when ctx_in is null
    const half_t* enc;     // [S, H]
    int enc_len;
    half_t* ctx_out[kDecMaxCtxOuts];
    int n_ctx_out;
    const half_t* cls_w;   // [vocab, H] or null
    const half_t* cls_b;   // [vocab] or null
    half_t* logits;        // [vocab]
    int vocab;
    unsigned int* hx;          // [kDecMaxLayers][NB][kDecEntryWords]
    unsigned int* g_counter;   // launches this buffer has seen, plus 1
    unsigned int* abort_flag;
    unsigned int* abort_host;
    unsigned int spin_limit;
    int H;
};

// Transpose-sum of four per-lane partial sums over the wavefront: lane l ends up with the total of slot
// 2 * (l & 1) + ((l >> 1) & 1), i.e. with slots {0, 2, 1, 3} in lanes {0, 1, 2, 3} (and every lane with lane & 3 alike).
__device__ __forceinline__ float transpose_sum4(const float (&acc)[4], int lane)
{
    const bool b0 = lane & 1, b1 = lane & 2;
    const float a0 = (b0 ? acc[2] : acc[0]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[0] : acc[2]);
    const float a1 = (b0 ? acc[3] : acc[1]) + dpp_mov_f32<kDppQuadXor1>(b0 ? acc[1] : acc[3]);
    const float a = (b1 ? a1 : a0) + dpp_mov_f32<kDppQuadXor2>(b1 ? a0 : a1);
    return wave_sum_mod4(a);
}

__global__ __launch_bounds__(kDecThreads) void decoder_step_f16_kernel(DecoderStepArgs p)
{
    __shared__ __align__(16) half_t in_vec[kDecMaxH];   // the current layer's input without the context part
    __shared__ __align__(16) half_t ctx_vec[kDecMaxH];
    __shared__ float comb[kDecUnits][4];                // gate sums of the second wavefront of each unit
    __shared__ __align__(8) unsigned short pub[kDecUnits];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int u = wave >> 1;   // unit of the block
    const int hf = wave & 1;   // which half of every row's columns
    const int H = p.H;
    const int nb = gridDim.x;
    const int j = blockIdx.x * kDecUnits + u;
    const bool unit_ok = j < H;
    const int jc = unit_ok ? j : H - 1;
    const int L = p.n_layers;
    const bool has_cls = p.cls_w != nullptr;

    const unsigned int g = __builtin_amdgcn_readfirstlane(__hip_atomic_load(p.g_counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    const unsigned short flag = (unsigned short)((g & 1u) << 14);

    // This wavefront's 16-byte piece of an H-wide row: pieces [0, n0) belong to half 0, [n0, nchunks) to half 1.
    const int nchunks = H >> 3;
    const int n0 = (nchunks + 1) >> 1;
    const int my_cnt = hf ? nchunks - n0 : n0;
    const bool active = lane < my_cnt;
    const int chunk = active ? (hf ? n0 : 0) + lane : 0;
    const int gate_of_slot[4] = {0, 2, 1, 3};
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;

    // ---- 0a. everything that does not wait for another layer: first W_hh of every layer and its h_prev ----
    half8_t w_a[kDecMaxLayers][4];
    half8_t hvec[kDecMaxLayers];
#pragma unroll
    for (int k = 0; k < kDecMaxLayers; ++k) {
        if (k < L) {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                w_a[k][v] = load_stream(reinterpret_cast<const half8_t*>(p.layer[k].w_hh + ((long)gate_of_slot[v] * H + jc) * H) + chunk);
            hvec[k] = active ? reinterpret_cast<const half8_t*>(p.layer[k].h_prev)[chunk] : zero8;
        }
    }

    // ---- 0b. the attention context, whole, in every block (S x H fp16 from the cache: cheaper than an exchange) ----
    bool any_ctx = false;
#pragma unroll
    for (int k = 0; k < kDecMaxLayers; ++k) any_ctx = any_ctx || (k < L && p.layer[k].takes_ctx);
    {
        const int col = tid * 2;
        if (col < H) {
            if (any_ctx || p.n_ctx_out > 0) {
                half2_t cv;
                if (p.ctx_in) {
                    cv = *reinterpret_cast<const half2_t*>(p.ctx_in + col);
                } else {
                    float c0 = 0.0f, c1 = 0.0f;
#pragma unroll 8
                    for (int e = 0; e < p.enc_len; ++e) {
                        const float a = (float)p.att[e];
                        const half2_t ev = *reinterpret_cast<const half2_t*>(p.enc + (long)e * H + col);
                        c0 = fmaf(a, (float)ev[0], c0);
                        c1 = fmaf(a, (float)ev[1], c1);
                    }
                    cv[0] = (half_t)c0;
                    cv[1] = (half_t)c1;
                }
                *reinterpret_cast<half2_t*>(&ctx_vec[col]) = cv;
                if ((col >> 2) == (int)blockIdx.x) {
                    for (int o = 0; o < p.n_ctx_out; ++o) *reinterpret_cast<half2_t*>(p.ctx_out[o] + col) = cv;
                }
            }
            // layer 0's input, for its residual sum (only defined when it is H wide)
            if (p.x_w == H) *reinterpret_cast<half2_t*>(&in_vec[col]) = *reinterpret_cast<const half2_t*>(p.x + col);
        }
    }
    __syncthreads();

    // ---- 0c. W_hh . h_prev ----
    float acc[kDecMaxLayers][4];
#pragma unroll
    for (int k = 0; k < kDecMaxLayers; ++k) {
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[k][v] = (k < L) ? dot8(w_a[k][v], hvec[k], 0.0f) : 0.0f;
    }

    // ---- 0d. the context columns of W_ih ----
    {
        const half8_t cvec = active ? *reinterpret_cast<const half8_t*>(&ctx_vec[chunk * 8]) : zero8;
#pragma unroll
        for (int k = 0; k < kDecMaxLayers; ++k) {
            if (k < L && p.layer[k].takes_ctx) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    w_a[k][v] = load_stream(reinterpret_cast<const half8_t*>(p.layer[k].w_ih + ((long)gate_of_slot[v] * H + jc) * p.layer[k].in_w + H) + chunk);
            }
        }
        // ---- 0f. the columns that wait for the layer before: into registers now, used after that layer's exchange ----
        half8_t w_dep[kDecMaxLayers - 1][4];
#pragma unroll
        for (int k = 1; k < kDecMaxLayers; ++k) {
            if (k < L) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    w_dep[k - 1][v] = load_stream(reinterpret_cast<const half8_t*>(p.layer[k].w_ih + ((long)gate_of_slot[v] * H + jc) * p.layer[k].in_w) + chunk);
            }
        }
        // ---- 0e. layer 0's own input columns (x is an argument of the step): any width, split between the halves ----
        {
            const int xw = p.layer[0].takes_ctx ? H : p.layer[0].in_w;
            const int xchunks = xw >> 3;
            const int x0 = (xchunks + 1) >> 1;
            const int begin = hf ? x0 : 0, end = hf ? xchunks : x0;
            const half8_t* xv = reinterpret_cast<const half8_t*>(p.x);
            for (int c = begin + lane; c < end; c += 64) {
                half8_t wr[4];
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    wr[v] = load_stream(reinterpret_cast<const half8_t*>(p.layer[0].w_ih + ((long)gate_of_slot[v] * H + jc) * p.layer[0].in_w) + c);
                const half8_t xr = xv[c];
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[0][v] = dot8(wr[v], xr, acc[0][v]);
            }
        }
#pragma unroll
        for (int k = 0; k < kDecMaxLayers; ++k) {
            if (k < L && p.layer[k].takes_ctx) {
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[k][v] = dot8(w_a[k][v], cvec, acc[k][v]);
            }
        }

        // ---- the layers, one exchange round each ----
        bool gave_up = false;
        half_t keep_h = (half_t)0.0f, keep_c = (half_t)0.0f;  // layer 0's new state, stored once every block has read h_prev
        const int my_gate = lane & 3;
#pragma unroll
        for (int k = 0; k < kDecMaxLayers; ++k) {
            if (k < L) {
                const DecoderLayerArgs& ly = p.layer[k];
                if (k > 0) {
                    const half8_t pv = active ? *reinterpret_cast<const half8_t*>(&in_vec[chunk * 8]) : zero8;
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[k][v] = dot8(w_dep[k - 1][v], pv, acc[k][v]);
                }
                float a = transpose_sum4(acc[k], lane);  // gate (lane & 3), this wavefront's half of the columns
                if (hf == 1 && lane < 4) comb[u][lane] = a;
                __syncthreads();
                if (hf == 0) {
                    a += comb[u][my_gate] + ly.bsum[(long)my_gate * H + jc];
                    const bool is_g = my_gate == 2;
                    const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
                    const float act = is_g ? 2.0f * sg - 1.0f : sg;
                    const float g_i = dpp_mov_f32<0x00>(act);
                    const float g_f = dpp_mov_f32<0x55>(act);
                    const float g_g = dpp_mov_f32<0xAA>(act);
                    const float g_o = dpp_mov_f32<0xFF>(act);
                    const float c_new = g_f * (float)ly.c_prev[jc] + g_i * g_g;
                    const half_t h_new = (half_t)(g_o * (2.0f * fast_sigmoid_f32(2.0f * c_new) - 1.0f));
                    if (lane == 0) {
                        const bool is_number = (c_new == c_new) && (g_o == g_o);
                        const unsigned short hbits = is_number ? __builtin_bit_cast(unsigned short, h_new) : kDecNanCode;
                        pub[u] = unit_ok ? (unsigned short)(hbits | flag) : flag;
                        if (unit_ok) {
                            const bool later = k == 0 && (L > 1 || has_cls);
                            if (later) {
                                keep_h = h_new;
                                keep_c = (half_t)c_new;
                            } else {
                                ly.hn[j] = h_new;
                                ly.cn[j] = (half_t)c_new;
                            }
                            if (ly.out) {
                                half_t o = h_new;
                                if (ly.residual) o = (half_t)((float)h_new + (float)(k == 0 ? p.x[j] : in_vec[j]));
                                ly.out[j] = o;
                            }
                        }
                    }
                }
                __syncthreads();
                if (k + 1 < L || has_cls) {
                    unsigned long long* slot = reinterpret_cast<unsigned long long*>(p.hx + ((long)k * nb) * kDecEntryWords);
                    if (tid == 0)
                        __hip_atomic_store(slot + (long)blockIdx.x * (kDecEntryWords / 2), *reinterpret_cast<const unsigned long long*>(&pub[0]),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (tid < nb) {
                        const unsigned long long want = flag ? 0x4000400040004000ull : 0ull;
                        unsigned long long word = 0ull;
                        unsigned int spins = 0;
                        while (true) {
                            word = __hip_atomic_load(slot + (long)tid * (kDecEntryWords / 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            if ((word & 0x4000400040004000ull) == want || gave_up) break;
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
                        // the four outputs of block `tid`; with a residual connection the next input is y + in
                        half4_t nv;
                        half4_t old;
#pragma unroll
                        for (int e = 0; e < 4; ++e) old[e] = in_vec[min(tid * 4 + e, kDecMaxH - 1)];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned short bits = (unsigned short)((word >> (16 * e)) & 0xbfffu);
                            half_t yv = __builtin_bit_cast(half_t, bits);
                            if ((bits & 0x7fffu) == kDecNanCode) yv = __builtin_bit_cast(half_t, (unsigned short)0x7e00u);
                            nv[e] = ly.residual ? (half_t)((float)yv + (float)old[e]) : yv;
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (tid * 4 + e < H) in_vec[tid * 4 + e] = nv[e];
                    }
                    __syncthreads();
                    if (k == 0 && hf == 0 && lane == 0 && unit_ok) {
                        // every block has published layer 0's output, so every block is past its reads of h_prev:
                        // hn / cn may be the very buffers h_prev / c_prev were read from
                        ly.hn[j] = keep_h;
                        ly.cn[j] = keep_c;
                    }
                }
            }
        }
    }

    // ---- the classifier: logits = W_c . out_last + b_c, rows dealt to the wavefronts of the whole grid four at a time ----
    if (has_cls) {
        const int gw = blockIdx.x * (kDecThreads / 64) + wave;
        const int nw = nb * (kDecThreads / 64);
        constexpr int CH = kDecMaxH / 8 / 64;  // 16-byte pieces of a row per lane
        half8_t vv[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) vv[c] = (c * 64 + lane < nchunks) ? *reinterpret_cast<const half8_t*>(&in_vec[(c * 64 + lane) * 8]) : zero8;
        const int V = p.vocab;
        for (long r0 = (long)gw * 4; r0 < V; r0 += (long)nw * 4) {
            half8_t wr[4][CH];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const long row = min(r0 + v, (long)V - 1);
                const half8_t* wp = reinterpret_cast<const half8_t*>(p.cls_w + row * H);
#pragma unroll
                for (int c = 0; c < CH; ++c) wr[v][c] = (c * 64 + lane < nchunks) ? load_stream(wp + c * 64 + lane) : zero8;
            }
            float s[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                s[v] = 0.0f;
#pragma unroll
                for (int c = 0; c < CH; ++c) s[v] = dot8(wr[v][c], vv[c], s[v]);
            }
            const float tot = transpose_sum4(s, lane);
            if (lane < 4) {
                const long row = r0 + gate_of_slot[lane];  // lane l holds slot {0, 2, 1, 3}[l]
                if (row < V) {
                    float r = tot;
                    if (p.cls_b) r += (float)p.cls_b[row];
                    p.logits[row] = (half_t)r;
                }
            }
        }
    }
    if (blockIdx.x == 0 && tid == 0) __hip_atomic_store(p.g_counter, g + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace pimhip
