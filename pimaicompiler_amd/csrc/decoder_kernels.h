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
// step is ONE persistent launch that streams every weight once, in layer order, as fast as memory delivers it, while
// the layers hand their outputs from block to block through a flagged exchange.
//
// The context columns of W_ih need not be streamed at all while the encoder outputs stay the same (every step of one
// sentence): W_ih[:, H:2H] . ctx = (W_ih[:, H:2H] . enc^T) . att, and the 4H x S matrix in brackets is computed once per
// sentence by the input-projection kernel (pimhip_decoder_plan_set_encoder).  A step then reads S values per gate row
// instead of H, and needs no context vector.  A caller that has the context instead passes it (ctx_in) and the columns
// are streamed.
//
// Grid: NB = ceil(H / 4) blocks (H <= 1024), all resident at once, of kDecStreamWaves + kDecPollWaves wavefronts each.
//   * Wavefronts 0..7 stream.  Block b owns hidden units 4b .. 4b+3 of every layer; two wavefronts share a unit and
//     split the columns of every weight row between them (lane l holds one 16-byte piece of each row).  Their
//     instruction stream holds no poll: loads return in order, so a poll behind a weight load could not be read before
//     that load has arrived.  Layer 0's weights go out first and its gate sums are delivered as soon as they arrive;
//     everything else that needs no other layer (W_hh . h_prev, the context term) is consumed as it arrives while layer
//     0's output travels, and the columns that wait for the layer before sit in registers until that layer's output is
//     there.  Each layer's four gate sums (slot v holds gate {i, g, f, o}[v], so that the transpose-sum leaves gate k in
//     lane k) are left in LDS.
//   * The other wavefronts hold no weights.  The first of them adds the partial sums of the block's four units,
//     applies the gates (lanes 4u .. 4u+3 = the gates of unit u), stores the state and publishes the block's four
//     outputs with one 8-byte store; all of them poll the other blocks' entries and put the layer's whole output into
//     LDS for the streamers.
// Three barriers per layer: gate sums ready (B1), the block's output stored (B2), next input ready (B3).  All wavefronts
// of a CU share its path to memory, and a request is served after every request issued before it: a store or a poll
// issued while weights are still queued is slow.  B2 lets the store and the first polls go out in front; what the
// streaming wavefronts ask for after it (one group of classifier rows per layer) streams while the output travels.
//
// Exchange: hx[stage][NB] entries of 64 bytes: a block's four fp16 outputs of layer `stage` in the first 8 bytes.
// |y| <= 1, so bit 14 of each fp16 carries a flag, the parity of the launch count g (kept per block in device memory: read at the
// start, advanced at the end): a slot written by launch g - 1 cannot pass for launch g, and the buffer starts as
// zeros with g = 1.  A NaN (bit 14 set) travels as the otherwise unused pattern 0x3fff.
//
// Every wait is bounded (`spin_limit` polls, one second of the constant clock), and a wait that gives up costs time, not
// the result.  The polling wavefront computes the entries that have not come itself, with the very operations, in the very
// order, of the block that owns them (dec_substitute): it holds every layer's previous state in LDS from the start of the
// kernel, so the values, and everything made of them, are bit for bit what they would have been.  The block that is late
// still does its own share when it runs.  The previous state may be the very buffers the new one goes to (hn == h_prev):
// a block that went past layer 0's exchange without everybody's entry cannot know whether everybody has read its inputs
// yet, so it parks its new state in the plan's memory instead; every block notes when it has read the inputs and when its
// parked state is complete, and whichever of these notes comes last makes its writer store the parked state to hn / cn.
#pragma once

#include "device_common.h"
#include "lstm_kernels.h"

namespace pimhip
{
// The barriers between the phases of a step: this wavefront's LDS traffic done, then s_barrier.  Nothing that passes between
// the wavefronts of a workgroup goes through global memory, and __syncthreads() would also wait until every global load
// and store the wavefront has in flight has come back (classifier rows asked for ahead, the state on its way to memory),
// which cost 0.7 us of a 26 us step.  What B2 needs is that the block's output is ISSUED in front of the loads that
// follow it, which the barrier gives either way.
__device__ __forceinline__ void dec_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

static constexpr int kDecMaxLayers = 4;
static constexpr int kDecStreamWaves = 8;
static constexpr int kDecPollWaves = 4;      // 1, 2 or 4: each lane polls 4 / kDecPollWaves entries (measured alike)
static constexpr int kDecThreads = 64 * (kDecStreamWaves + kDecPollWaves);
static constexpr int kDecUnits = 4;          // hidden units per block
static constexpr int kDecMaxH = 1024;        // 2 wavefronts x 64 lanes x 8 columns per row
static constexpr int kDecEntryWords = 16;    // 32-bit words between the entries of consecutive blocks (64 bytes)
static constexpr int kDecStages = kDecMaxLayers;      // exchange stages: one per layer
static constexpr int kDecMaxCtxOuts = 4;
static constexpr unsigned short kDecNanCode = 0x3fffu;
static constexpr int kDecNoteWords = 8;
static constexpr unsigned int kDecImpatientPolls = 4096u;  // the poll limit of a wavefront's waits after its first one that gave up

struct DecoderLayerArgs {
    const half_t* w_ih;    // [4H, in_w]
    const half_t* w_hh;    // [4H, H]
    const float* bsum;     // [4H] fp32, b_ih + b_hh
    const float* cx_proj;  // [4H, S] fp32 = W_ih[:, H:2H] . enc^T, or null: then the context columns are streamed (ctx_in)
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
    const half_t* att;     // [S] attention weights (with cx_proj; and for ctx_out)
    const half_t* enc;     // [S, H] encoder outputs, only read for ctx_out
    int enc_len;           // S
    half_t* ctx_out[kDecMaxCtxOuts];
    int n_ctx_out;
    const half_t* cls_w;   // [vocab, H] or null
    const half_t* cls_b;   // [vocab] or null
    half_t* logits;        // [vocab]
    int vocab;
    unsigned int* hx;          // [kDecStages][NB][kDecEntryWords]
    // Per block b, kDecNoteWords 64-bit words (one 64-byte line) at notes + b * kDecNoteWords, written by that block only:
    //   [0] the launches the block has run (every block runs once per launch, so all agree: this launch is number g = that + 1)
    //   [1] the last launch in which the block has read all the inputs of the step
    //   [2] the last launch in which the block parked its new state (written when all of it is in place)
    // and after the blocks' lines one word: the last launch in which some block parked its new state.  All zero at first.
    unsigned long long* notes;
    half_t* parked_h;          // [n_layers][H] the parked h of such blocks
    half_t* parked_c;          // [n_layers][H]
    unsigned int* abort_host;  // pinned host word: raised when a wait gives up, for the host's count
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

__device__ __forceinline__ unsigned int readlane_u32(unsigned int v, int l)
{
    return (unsigned int)__builtin_amdgcn_readlane((int)v, l);
}

// The cell of one hidden unit from its four gate sums: lanes 4q .. 4q+3 of a quad hold the sums of the gates i, f, g, o
// (`pg` = lane & 3), every lane of the quad returns the unit's h.  The owner of a unit and a block that stands in for it
// both go through here; every operation is spelled out (no contraction left to the compiler) so that both get the same bits.
__device__ __forceinline__ half_t dec_cell(float a, int pg, float cprev, float& c_new, bool& is_number)
{
    const bool is_g = pg == 2;
    const float sg = fast_sigmoid_f32(is_g ? 2.0f * a : a);
    const float act = is_g ? fmaf(2.0f, sg, -1.0f) : sg;
    const float g_i = dpp_mov_f32<0x00>(act);
    const float g_f = dpp_mov_f32<0x55>(act);
    const float g_g = dpp_mov_f32<0xAA>(act);
    const float g_o = dpp_mov_f32<0xFF>(act);
    c_new = fmaf(g_f, cprev, g_i * g_g);
    is_number = (c_new == c_new) && (g_o == g_o);
    return round_f16(g_o * fmaf(2.0f, fast_sigmoid_f32(2.0f * c_new), -1.0f));
}

// How a streaming wavefront (unit `j`, half `hf` of the columns) splits a row of `nchunks` 16-byte pieces.
struct DecPiece {
    bool active;
    int chunk;
};
__device__ __forceinline__ DecPiece dec_piece(int nchunks, int hf, int lane)
{
    const int n0 = (nchunks + 1) >> 1;
    const int my_cnt = hf ? nchunks - n0 : n0;
    DecPiece r;
    r.active = lane < my_cnt;
    r.chunk = r.active ? (hf ? n0 : 0) + lane : 0;
    return r;
}

// The exchange entry of block `z` for layer `k` (first: k == 0), made by one wavefront from the step's inputs and the
// layer's input: the same loads, products and sums, in the same order, as block z's own wavefronts make (two streaming
// wavefronts per unit, then the cell), so the same bits.  hprev_k / cprev_k: the layer's previous state, all H values;
// in_vec: the layer's input without the context part (k >= 1); ctx_vec: a given context.
// (Inlined: as a function of its own it needs a stack, which costs the undisturbed step more than the cold code in its way.)
struct DecSubstituteLayer {
    const half_t* w_ih;
    const half_t* w_hh;
    const float* bsum;
    const float* cx_proj;
    int in_w;
    int takes_ctx;
};
__device__ __forceinline__ unsigned long long dec_substitute(const DecSubstituteLayer ly, bool first, int z, int lane, int H,
                                                                       const half_t* x, const half_t* att, int S, bool ctx_given,
                                                                       const half_t* hprev_k, const half_t* cprev_k,
                                                                       const half_t* in_vec, const half_t* ctx_vec, unsigned short flag)
{
    const int nchunks = H >> 3;
    const int gate_of_slot[4] = {0, 2, 1, 3};
    const int pg = lane & 3;
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;
    unsigned long long word = 0ull;
    for (int u = 0; u < kDecUnits; ++u) {
        const int j = z * kDecUnits + u;
        unsigned int bits = flag;
        if (j < H) {
            float half_sum[2];
            for (int hf = 0; hf < 2; ++hf) {
                const DecPiece pc = dec_piece(nchunks, hf, lane);
                auto row_ptr = [&](const half_t* base, int v, long pitch, long col0) {
                    return reinterpret_cast<const half8_t*>(base + ((long)gate_of_slot[v] * H + j) * pitch + col0);
                };
                float acc[4];
                const half8_t hv = pc.active ? *reinterpret_cast<const half8_t*>(&hprev_k[pc.chunk * 8]) : zero8;
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[v] = dot8(load_stream(row_ptr(ly.w_hh, v, H, 0) + pc.chunk), hv, 0.0f);
                if (ly.takes_ctx) {
                    if (ly.cx_proj) {
                        const int e_mine = 64 * hf + lane;
                        const float att_mine = (att && e_mine < S) ? (float)att[e_mine] : 0.0f;
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            acc[v] = fmaf(att_mine, ly.cx_proj[((long)gate_of_slot[v] * H + j) * S + min(e_mine, S - 1)], acc[v]);
                        for (int e = e_mine + 128; e < S; e += 128) {
                            const float a = (float)att[e];
#pragma unroll
                            for (int v = 0; v < 4; ++v) acc[v] = fmaf(a, ly.cx_proj[((long)gate_of_slot[v] * H + j) * S + e], acc[v]);
                        }
                    } else {
                        const half8_t cvec = (ctx_given && pc.active) ? *reinterpret_cast<const half8_t*>(&ctx_vec[pc.chunk * 8]) : zero8;
#pragma unroll
                        for (int v = 0; v < 4; ++v) acc[v] = dot8(load_stream(row_ptr(ly.w_ih, v, ly.in_w, H) + pc.chunk), cvec, acc[v]);
                    }
                }
                if (first) {
                    const int xw = ly.takes_ctx ? H : ly.in_w;
                    const int xchunks = xw >> 3;
                    const int xn0 = (xchunks + 1) >> 1;
                    const int x_begin = hf ? xn0 : 0, x_end = hf ? xchunks : xn0;
                    const half8_t* xv = reinterpret_cast<const half8_t*>(x);
                    if (x_end - x_begin <= 64) {
                        const bool x_active = lane < x_end - x_begin;
                        const int x_chunk = x_active ? x_begin + lane : 0;
                        const half8_t xvec = x_active ? xv[x_chunk] : zero8;
#pragma unroll
                        for (int v = 0; v < 4; ++v) acc[v] = dot8(load_stream(row_ptr(ly.w_ih, v, ly.in_w, 0) + x_chunk), xvec, acc[v]);
                    } else {
                        for (int c = x_begin + lane; c < x_end; c += 64) {
                            const half8_t xr = xv[c];
#pragma unroll
                            for (int v = 0; v < 4; ++v) acc[v] = dot8(load_stream(row_ptr(ly.w_ih, v, ly.in_w, 0) + c), xr, acc[v]);
                        }
                    }
                } else {
                    const half8_t pv = pc.active ? *reinterpret_cast<const half8_t*>(&in_vec[pc.chunk * 8]) : zero8;
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[v] = dot8(load_stream(row_ptr(ly.w_ih, v, ly.in_w, 0) + pc.chunk), pv, acc[v]);
                }
                half_sum[hf] = transpose_sum4(acc, lane);  // gate (lane & 3) in every lane
            }
            const float a = half_sum[0] + half_sum[1] + ly.bsum[(long)pg * H + j];
            float c_new;
            bool is_number;
            const half_t h_new = dec_cell(a, pg, (float)cprev_k[j], c_new, is_number);
            // Lanes 0..3 hold what the owner's cell works on: the sums the streaming wavefronts hand over are those of their
            // lanes 0..3, and the other quads of a wavefront add the same four partial sums in another order (wave_sum_mod4).
            bits = readlane_u32((unsigned int)((is_number ? __builtin_bit_cast(unsigned short, h_new) : kDecNanCode) | flag), 0);
        }
        word |= (unsigned long long)bits << (16 * u);
    }
    return word;
}

// L = p.n_layers and CLS = "there is a classifier" are template parameters so that the order of loads and uses is fixed
// at compile time: the lifetime of every register, and the number of later loads that may still be in flight when an
// earlier one is waited for (a load issued under a run-time condition would make every such wait a wait for all).
// How many groups of classifier rows (four rows per streaming wavefront each; a wavefront's registers hold four groups)
// are asked for right after layer k's output has been stored.  One group stands in front of each exchange's polls: the
// 16 MB stream while the output travels.  (Measured on MI355X, four layers, 32000 rows: {1, 1, 1, 1} 26.7 us per step;
// {2, 0, 0, 2} 30.3 us; {0, 2, 0, 2} 30.3 us; {0, 1, 1, 2} 27.3 us; {0, 1, 2, 1} 27.3 us; {1, 1, 2, 0} 31.0 us.)
template <int L>
__device__ constexpr int cls_groups_after(int k)
{
    if (k + 1 == L) return 4;  // whatever is left
    if (L == 2) return 2;
    if (L == 3) return k == 0 ? 1 : 2;
    return k <= 2 ? 1 : 0;
}

template <int L, bool CLS>
__global__ __launch_bounds__(kDecThreads) void decoder_step_f16_kernel(DecoderStepArgs p)
{
    static_assert(L >= 1 && L <= kDecMaxLayers, "layers per step");
    static_assert(kDecPollWaves == 1 || kDecPollWaves == 2 || kDecPollWaves == 4, "entries per polling lane");
    __shared__ __align__(16) half_t in_vec[2][kDecMaxH];               // layer k's input without the context part in [k & 1], its output goes to the other
    __shared__ __align__(16) half_t ctx_vec[kDecMaxH];                 // a given context (ctx_in)
    __shared__ __align__(16) half_t hprev[kDecMaxLayers][kDecMaxH];    // every layer's previous hidden state (the streamers read layer 0's from memory)
    __shared__ __align__(16) half_t cprev[kDecMaxLayers][kDecMaxH];    // every layer's previous cell state: for entries that have to be made here
    __shared__ unsigned int parked_lds;                                // some wavefront went past layer 0's exchange without every entry
    __shared__ float part[kDecStreamWaves][4];                         // a layer's gate sums: [wavefront][gate]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int H = p.H;
    const int nb = gridDim.x;
    constexpr bool has_cls = CLS;
    const int nchunks = H >> 3;
    bool any_ctx = false;
#pragma unroll
    for (int k = 0; k < L; ++k) any_ctx = any_ctx || p.layer[k].takes_ctx;
    // a first layer that takes a given context needs it in LDS before its first product (one barrier more, for every wavefront)
    const bool staged_ctx_first = p.ctx_in && p.layer[0].takes_ctx;
    half8_t zero8;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero8[e] = (half_t)0.0f;

    if (wave < kDecStreamWaves) {
        // =========================================== the streaming wavefronts ===========================================
        const int u = wave >> 1;   // unit of the block
        const int hf = wave & 1;   // which half of every row's columns
        const int j = blockIdx.x * kDecUnits + u;
        const int jc = j < H ? j : H - 1;
        // This wavefront's 16-byte piece of an H-wide row: pieces [0, n0) belong to half 0, [n0, nchunks) to half 1.
        const int n0 = (nchunks + 1) >> 1;
        const int my_cnt = hf ? nchunks - n0 : n0;
        const bool active = lane < my_cnt;
        const int chunk = active ? (hf ? n0 : 0) + lane : 0;
        const int gate_of_slot[4] = {0, 2, 1, 3};
        // layer 0's input without the context: any width, split between the two halves like the rows
        const int xw = p.layer[0].takes_ctx ? H : p.layer[0].in_w;
        const int xchunks = xw >> 3;
        const int xn0 = (xchunks + 1) >> 1;
        const int x_begin = hf ? xn0 : 0, x_end = hf ? xchunks : xn0;
        const bool x_one_piece = x_end - x_begin <= 64;
        const bool x_active = lane < x_end - x_begin;
        const int x_chunk = x_active ? x_begin + lane : 0;

        // Weights per layer, one 16-byte piece of each of the four gate rows per lane, in two groups:
        //   A(k): W_hh, the context term and, for layer 0, its input columns: what needs no other layer
        //   D(k): the input columns of W_ih of a layer k >= 1, which wait for layer k - 1's output
        half8_t w_hh[L][4], w_cx[L][4], w_in[L][4];
        float m_cx[L][4];  // projected context: this unit's four gate rows of the layer's 4H x S matrix at position e_mine
        half8_t xvec = zero8;
        // the two wavefronts of a unit take alternate runs of 64 encoder positions: lane l the position 64 hf + l (+ 128 i)
        const int S = p.enc_len;
        const int e_mine = 64 * hf + lane;
        const float att_mine = (any_ctx && p.att && e_mine < S) ? (float)p.att[e_mine] : 0.0f;
        auto row_ptr = [&](const half_t* base, int v, long pitch, long col0) {
            return reinterpret_cast<const half8_t*>(base + ((long)gate_of_slot[v] * H + jc) * pitch + col0);
        };
        auto issue_a = [&](int k) __attribute__((always_inline)) {
            const DecoderLayerArgs& ly = p.layer[k];
#pragma unroll
            for (int v = 0; v < 4; ++v) w_hh[k][v] = load_stream(row_ptr(ly.w_hh, v, H, 0) + chunk);
            if (ly.takes_ctx) {
                if (ly.cx_proj) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) m_cx[k][v] = ly.cx_proj[((long)gate_of_slot[v] * H + jc) * S + min(e_mine, S - 1)];
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v) w_cx[k][v] = load_stream(row_ptr(ly.w_ih, v, ly.in_w, H) + chunk);
                }
            }
            if (k == 0 && x_one_piece) {
#pragma unroll
                for (int v = 0; v < 4; ++v) w_in[0][v] = load_stream(row_ptr(ly.w_ih, v, ly.in_w, 0) + x_chunk);
                if (x_active) xvec = reinterpret_cast<const half8_t*>(p.x)[x_chunk];
            }
        };
        auto issue_d = [&](int k) __attribute__((always_inline)) {
            const DecoderLayerArgs& ly = p.layer[k];
#pragma unroll
            for (int v = 0; v < 4; ++v) w_in[k][v] = load_stream(row_ptr(ly.w_ih, v, ly.in_w, 0) + chunk);
        };

        // The classifier's rows are dealt to the streaming wavefronts of the whole grid four at a time.  A wavefront's first
        // groups are fetched behind the layers' weights, the next ones as soon as the last layer's registers are free.
        constexpr int CH = kDecMaxH / 8 / 64;  // 16-byte pieces of a classifier row per lane
        const int gw = blockIdx.x * kDecStreamWaves + wave;
        const int nw = nb * kDecStreamWaves;
        const int V = p.vocab;
        half8_t cbuf[4][4][CH];
        auto cls_row0 = [&](int it) { return ((long)it * nw + gw) * 4; };
        auto cls_issue = [&](half8_t (&dst)[4][CH], int it) __attribute__((always_inline)) {
            const long r0 = cls_row0(it);
            if (has_cls) {  // (rows past the end are clamped, loaded and dropped: the count of loads in flight stays fixed)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const long row = min(r0 + v, (long)V - 1);
                    const half8_t* wp = reinterpret_cast<const half8_t*>(p.cls_w + row * H);
#pragma unroll
                    for (int c = 0; c < CH; ++c) dst[v][c] = load_stream(wp + min(c * 64 + lane, nchunks - 1));
                }
            }
        };
        float acc[L][4];
        auto consume_a = [&](int k, const half8_t& cvec, const half8_t& hv) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[k][v] = dot8(w_hh[k][v], hv, 0.0f);
            if (p.layer[k].takes_ctx) {
                if (p.layer[k].cx_proj) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[k][v] = fmaf(att_mine, m_cx[k][v], acc[k][v]);
                    for (int e = e_mine + 128; e < S; e += 128) {  // more than 128 encoder positions
                        const float a = (float)p.att[e];
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            acc[k][v] = fmaf(a, p.layer[k].cx_proj[((long)gate_of_slot[v] * H + jc) * S + e], acc[k][v]);
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[k][v] = dot8(w_cx[k][v], cvec, acc[k][v]);
                }
            }
        };
        auto deliver = [&](int k) __attribute__((always_inline)) {
            const float a = transpose_sum4(acc[k], lane);  // gate (lane & 3), this wavefront's half of the columns
            if (lane < 4) part[wave][lane] = a;
            dec_barrier();  // B1: the gate sums of layer k are in LDS
        };

        // Layer 0 waits for nothing but its own weights: its h_prev comes straight from memory, ahead of them.
        const half8_t hv0 = active ? reinterpret_cast<const half8_t*>(p.layer[0].h_prev)[chunk] : zero8;
        issue_a(0);
        // the bias of this wavefront's first sixteen classifier rows, long before the end of the step needs it
        // (every lane loads, from a clamped row: a load under a run-time condition would blur the count of loads in flight)
        float cls_bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (has_cls) {
            const half_t* bias_src = p.cls_b ? p.cls_b : p.cls_w;
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const long row = min(cls_row0(it) + gate_of_slot[lane & 3], (long)V - 1);
                const float b = (float)bias_src[row];
                cls_bias[it] = p.cls_b ? b : 0.0f;
            }
        }
        if (staged_ctx_first) dec_barrier();  // B0: a given context is in LDS (a first layer that takes it)
        half8_t cvec = (staged_ctx_first && active) ? *reinterpret_cast<const half8_t*>(&ctx_vec[chunk * 8]) : zero8;
        consume_a(0, cvec, hv0);
        if (x_one_piece) {
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[0][v] = dot8(w_in[0][v], xvec, acc[0][v]);
        } else {
            // a first layer with a wide plain input: its columns in a loop
            const half8_t* xv = reinterpret_cast<const half8_t*>(p.x);
            for (int c = x_begin + lane; c < x_end; c += 64) {
                half8_t wr[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) wr[v] = load_stream(row_ptr(p.layer[0].w_ih, v, p.layer[0].in_w, 0) + c);
                const half8_t xr = xv[c];
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[0][v] = dot8(wr[v], xr, acc[0][v]);
            }
        }
        deliver(0);
        // B2: the block's output is on its way before anything else is asked for.  A store, and the polls behind it, wait in
        // the CU's memory pipeline for every load issued before them; without this barrier layer 0's output left some
        // blocks 5 us late (behind 24 MB of the later layers' rows) and every block waited for it.
        if (L > 1 || has_cls) dec_barrier();
        // everything else that needs no other layer goes out now and is consumed as it arrives, while layer 0's output travels
#pragma unroll
        for (int k = 1; k < L; ++k) issue_a(k);
        // (after B1 of layer 0: every later layer's h_prev and a given context are in LDS)
        if (p.ctx_in && active) cvec = *reinterpret_cast<const half8_t*>(&ctx_vec[chunk * 8]);
        auto hv_of = [&](int k) { return active ? *reinterpret_cast<const half8_t*>(&hprev[k][chunk * 8]) : zero8; };
        // The registers freed by each consumed group take the next loads: D(1..), then classifier rows, of which a
        // wavefront's first four groups go out at fixed points (cls_groups_after).
        int cls_next = 0;  // (a compile-time value at every use: the code below is straight-line in L)
        auto cls_prefetch = [&](int n) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i < n && cls_next < 4) {
                    if (cls_next == 0) cls_issue(cbuf[0], 0);
                    if (cls_next == 1) cls_issue(cbuf[1], 1);
                    if (cls_next == 2) cls_issue(cbuf[2], 2);
                    if (cls_next == 3) cls_issue(cbuf[3], 3);
                    ++cls_next;
                }
            }
        };
        if (L >= 2) {
            consume_a(1, cvec, hv_of(1));
            issue_d(1);
            if (L >= 3) issue_d(2);
        }
        if (L >= 3) {
            consume_a(2, cvec, hv_of(2));
            if (L >= 4) issue_d(3);
        }
        if (L >= 4) consume_a(3, cvec, hv_of(3));
        cls_prefetch(cls_groups_after<L>(0));
        if (L > 1 || has_cls) {
            dec_barrier();  // B3 of layer 0: its whole output (the next input) is in LDS
        }
#pragma unroll
        for (int k = 1; k < L; ++k) {
            const half8_t pv = active ? *reinterpret_cast<const half8_t*>(&in_vec[k & 1][chunk * 8]) : zero8;
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[k][v] = dot8(w_in[k][v], pv, acc[k][v]);
            deliver(k);
            // B2 again, then the next classifier rows: they stream while this layer's output travels
            if (has_cls && cls_groups_after<L>(k) > 0) dec_barrier();
            cls_prefetch(cls_groups_after<L>(k));
            if (k + 1 < L || has_cls) {
                dec_barrier();  // B3: the layer's whole output (the next input) is in LDS
            }
        }

        // ---- the classifier: logits = W_c . out_last + b_c ----
        if (has_cls) {
            half8_t vv[CH];
#pragma unroll
            for (int c = 0; c < CH; ++c) vv[c] = (c * 64 + lane < nchunks) ? *reinterpret_cast<const half8_t*>(&in_vec[L & 1][(c * 64 + lane) * 8]) : zero8;
            auto cls_finish = [&](const half8_t (&src)[4][CH], int it, float bias, bool bias_given) __attribute__((always_inline)) {
                const long r0 = cls_row0(it);
                float s[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    s[v] = 0.0f;
#pragma unroll
                    for (int c = 0; c < CH; ++c) s[v] = dot8(src[v][c], vv[c], s[v]);
                }
                const float tot = transpose_sum4(s, lane);
                if (lane < 4) {
                    const long row = r0 + gate_of_slot[lane];  // lane l holds slot {0, 2, 1, 3}[l]
                    if (row < V) {
                        float r = tot + bias;
                        if (!bias_given && p.cls_b) r += (float)p.cls_b[row];
                        p.logits[row] = (half_t)r;
                    }
                }
            };
            cls_finish(cbuf[0], 0, cls_bias[0], true);
            cls_finish(cbuf[1], 1, cls_bias[1], true);
            cls_finish(cbuf[2], 2, cls_bias[2], true);
            cls_finish(cbuf[3], 3, cls_bias[3], true);
            for (int it = 4; cls_row0(it) < V; it += 2) {  // vocabularies beyond 16 rows per wavefront: two groups at a time
                cls_issue(cbuf[0], it);
                cls_issue(cbuf[1], it + 1);
                cls_finish(cbuf[0], it, 0.0f, false);
                cls_finish(cbuf[1], it + 1, 0.0f, false);
            }
        }
    } else {
        // ========================= the wavefronts that activate, publish and poll (no weights) =========================
        const int pw = wave - kDecStreamWaves;         // 0: also activates and publishes
        constexpr int QP = 4 / kDecPollWaves;          // entries polled per lane: blocks lane + 64 (pw * QP + q)
        // the number of this launch, kept per block: a block that runs late must not find it advanced by one that is done
        unsigned long long* const my_notes = p.notes + (long)blockIdx.x * kDecNoteWords;
        unsigned long long* const parked_any = p.notes + (long)nb * kDecNoteWords;
        const unsigned long long g = __hip_atomic_load(my_notes, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1ull;
        if (tid == kDecStreamWaves * 64) parked_lds = 0u;
        // lanes 4u .. 4u+3 are the gates i, f, g, o of unit u of this block (lanes 16.. repeat them)
        const int pu = (lane >> 2) & 3, pg = lane & 3;
        const int pj = blockIdx.x * kDecUnits + pu;
        const bool p_ok = pj < H;
        const int pjc = p_ok ? pj : H - 1;
        const bool owner = pw == 0 && pg == 0 && lane < 16 && p_ok;
        float bias_r[L], cprev_r[L];
#pragma unroll
        for (int k = 0; k < L; ++k) {
            bias_r[k] = cprev_r[k] = 0.0f;
            if (pw == 0) {
                bias_r[k] = p.layer[k].bsum[(long)pg * H + pjc];
                cprev_r[k] = (float)p.layer[k].c_prev[pjc];
            }
        }
        // every layer's previous state, layer 0's input (for its residual sum, when it is H wide) and a given context into LDS
        for (int c = pw * 64 + lane; c < nchunks; c += 64 * kDecPollWaves) {
#pragma unroll
            for (int k = 0; k < L; ++k) {
                *reinterpret_cast<half8_t*>(&hprev[k][c * 8]) = reinterpret_cast<const half8_t*>(p.layer[k].h_prev)[c];
                *reinterpret_cast<half8_t*>(&cprev[k][c * 8]) = reinterpret_cast<const half8_t*>(p.layer[k].c_prev)[c];
            }
            if (p.x_w == H) *reinterpret_cast<half8_t*>(&in_vec[0][c * 8]) = reinterpret_cast<const half8_t*>(p.x)[c];
            if (p.ctx_in) *reinterpret_cast<half8_t*>(&ctx_vec[c * 8]) = reinterpret_cast<const half8_t*>(p.ctx_in)[c];
        }
        const unsigned short flag = (unsigned short)((g & 1u) << 14);
        bool gave_up = false;  // a wait of this wavefront has given up: its later waits are short
        // one step of a bounded wait: true when the caller should stop waiting
        unsigned long long t_first = 0ull;
        auto give_up_check = [&](unsigned int& spins) {
            ++spins;
            if ((spins & 255u) == 0u && wait_clock_expired(spins, t_first)) spins = 0xffffffffu;  // gives up below
            const unsigned int limit = gave_up ? min(p.spin_limit, kDecImpatientPolls) : p.spin_limit;
            if (spins < limit) return false;
            __hip_atomic_store(p.abort_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            gave_up = true;
            return true;
        };
        // Parked state goes to hn / cn once every block has read the step's inputs (every block notes that, after layer 0's
        // gate sums) and the state is all there (its block notes that, at its end).  Each side writes its note, then looks
        // at the other's: whichever comes last sees both and does the stores (twice the same values if both do).
        auto store_parked = [&]() {
            __threadfence();
            bool all_read = true;
            for (int z = lane; z < nb; z += 64)
                all_read = all_read && __hip_atomic_load(p.notes + (long)z * kDecNoteWords + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == g;
            if (__ballot(!all_read) != 0ull) return;
            for (int z = lane; z < nb; z += 64) {
                if (__hip_atomic_load(p.notes + (long)z * kDecNoteWords + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != g) continue;
                __threadfence();
                for (int k = 0; k < L; ++k) {
                    for (int u = 0; u < kDecUnits; ++u) {
                        const int j = z * kDecUnits + u;
                        if (j < H) {
                            p.layer[k].hn[j] = p.parked_h[(long)k * H + j];
                            p.layer[k].cn[j] = p.parked_c[(long)k * H + j];
                        }
                    }
                }
            }
        };
        constexpr int kLastExchange = has_cls ? L - 1 : L - 2;  // the last exchange of the step
        bool parked = false;  // this block keeps its new state in the plan's memory instead of hn / cn
        unsigned long long parked_seen = 0ull;

        // ---- where the caller wants the attention context stored, this block stores its own four columns ----
        if (pw == 0 && p.n_ctx_out > 0 && blockIdx.x * kDecUnits + kDecUnits <= H) {
            const int col0 = blockIdx.x * kDecUnits;
            if (p.ctx_in) {
                if (lane < 2) {
                    for (int o = 0; o < p.n_ctx_out; ++o)
                        *reinterpret_cast<half2_t*>(p.ctx_out[o] + col0 + 2 * lane) = *reinterpret_cast<const half2_t*>(p.ctx_in + col0 + 2 * lane);
                }
            } else {
                float cs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                for (int e = lane; e < p.enc_len; e += 64) {
                    const float a = (float)p.att[e];
                    const half2_t e01 = *reinterpret_cast<const half2_t*>(p.enc + (long)e * H + col0);
                    const half2_t e23 = *reinterpret_cast<const half2_t*>(p.enc + (long)e * H + col0 + 2);
                    cs[0] = fmaf(a, (float)e01[0], cs[0]);
                    cs[1] = fmaf(a, (float)e01[1], cs[1]);
                    cs[2] = fmaf(a, (float)e23[0], cs[2]);
                    cs[3] = fmaf(a, (float)e23[1], cs[3]);
                }
                const float tot = transpose_sum4(cs, lane);  // lanes 0..3 hold columns {0, 2, 1, 3}
                const unsigned int mine = (unsigned int)__builtin_bit_cast(unsigned short, (half_t)tot);
                const unsigned int c0 = readlane_u32(mine, 0), c1 = readlane_u32(mine, 2), c2 = readlane_u32(mine, 1), c3 = readlane_u32(mine, 3);
                if (lane < 2) {
                    half2_t cv;
                    cv[0] = __builtin_bit_cast(half_t, (unsigned short)(lane == 0 ? c0 : c2));
                    cv[1] = __builtin_bit_cast(half_t, (unsigned short)(lane == 0 ? c1 : c3));
                    for (int o = 0; o < p.n_ctx_out; ++o) *reinterpret_cast<half2_t*>(p.ctx_out[o] + col0 + 2 * lane) = cv;
                }
            }
        }
        if (staged_ctx_first) dec_barrier();  // B0

        half_t keep_h = (half_t)0.0f, keep_c = (half_t)0.0f;  // layer 0's new state, stored once every block has read h_prev
#pragma unroll
        for (int k = 0; k < L; ++k) {
            const DecoderLayerArgs& ly = p.layer[k];
            dec_barrier();  // B1: the gate sums of layer k are in LDS
            const bool exchange = k + 1 < L || has_cls;
            if (k == 0 && kLastExchange >= 0 && tid == kDecThreads - 64) {
                // every wavefront of the block is past its reads of the step's inputs (the streamers have used h_prev of
                // layer 0, the others have filled LDS): noted for whoever has parked state to store
                __hip_atomic_store(my_notes + 1, g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (pw == 0) {
                // (the streamers leave gate k in lane k, i.e. in part[.][k])
                const float a = part[2 * pu][pg] + part[2 * pu + 1][pg] + bias_r[k];
                float c_new;
                bool is_number;
                const half_t h_new = dec_cell(a, pg, cprev_r[k], c_new, is_number);
                half_t* const dst_h = parked ? p.parked_h + (long)k * H : ly.hn;
                half_t* const dst_c = parked ? p.parked_c + (long)k * H : ly.cn;
                const unsigned int hbits = p_ok ? (unsigned int)((is_number ? __builtin_bit_cast(unsigned short, h_new) : kDecNanCode) | flag)
                                                : (unsigned int)flag;
                if (owner) {
                    if (k == 0 && exchange) {
                        keep_h = h_new;
                        keep_c = round_f16(c_new);
                    } else {
                        dst_h[pj] = h_new;
                        dst_c[pj] = round_f16(c_new);
                    }
                    if (ly.out) {
                        half_t o = h_new;
                        if (ly.residual) o = (half_t)((float)h_new + (float)in_vec[k & 1][pj]);
                        ly.out[pj] = o;
                    }
                }
                if (exchange) {
                    unsigned long long* slot = reinterpret_cast<unsigned long long*>(p.hx + ((long)k * nb) * kDecEntryWords);
                    const unsigned long long word = (unsigned long long)readlane_u32(hbits, 0) | ((unsigned long long)readlane_u32(hbits, 4) << 16) |
                                                    ((unsigned long long)readlane_u32(hbits, 8) << 32) | ((unsigned long long)readlane_u32(hbits, 12) << 48);
                    if (lane == 0)
                        __hip_atomic_store(slot + (long)blockIdx.x * (kDecEntryWords / 2), word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            if (k == 0 ? (L > 1 || has_cls) : (has_cls && cls_groups_after<L>(k) > 0)) dec_barrier();  // B2: this block's output has been stored
            if (exchange) {
                const unsigned long long* slot = reinterpret_cast<const unsigned long long*>(p.hx + ((long)k * nb) * kDecEntryWords);
                const unsigned long long want = flag ? 0x4000400040004000ull : 0ull;
                unsigned long long got[QP];
#pragma unroll
                for (int q = 0; q < QP; ++q) got[q] = want;
                unsigned int spins = 0;
                while (true) {
                    bool ok = true;
#pragma unroll
                    for (int q = 0; q < QP; ++q) {
                        const int blk = lane + 64 * (pw * QP + q);
                        if (blk < nb)
                            got[q] = __hip_atomic_load(const_cast<unsigned long long*>(slot) + (long)blk * (kDecEntryWords / 2), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int q = 0; q < QP; ++q) ok = ok && (got[q] & 0x4000400040004000ull) == want;
                    if (ok || give_up_check(spins)) break;
                }
                // Entries that have not come: made here, bit for bit as their owners make them.
#pragma unroll
                for (int q = 0; q < QP; ++q) {
                    const int blk = lane + 64 * (pw * QP + q);
                    unsigned long long missing = __ballot(blk < nb && (got[q] & 0x4000400040004000ull) != want);
                    if (missing != 0ull && k == 0 && lane == 0) parked_lds = 1u;
                    while (__builtin_expect(missing != 0ull, 0)) {  // (said to be unlikely: 0.3 us of the undisturbed step)
                        const int src = __builtin_ctzll(missing);
                        missing &= missing - 1ull;
                        const DecSubstituteLayer sl = {ly.w_ih, ly.w_hh, ly.bsum, ly.cx_proj, ly.in_w, ly.takes_ctx};
                        const unsigned long long word = dec_substitute(sl, k == 0, src + 64 * (pw * QP + q), lane, H, p.x, p.att, p.enc_len, p.ctx_in != nullptr,
                                                                       hprev[k], cprev[k], in_vec[k & 1], ctx_vec, flag);
                        if (lane == src) got[q] = word;
                    }
                }
                // the outputs of this lane's blocks; with a residual connection the next input is y + in
#pragma unroll
                for (int q = 0; q < QP; ++q) {
                    const int blk = lane + 64 * (pw * QP + q);
                    if (blk < nb) {
                        const half4_t old = *reinterpret_cast<const half4_t*>(&in_vec[k & 1][blk * 4]);
                        half4_t nv;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned short bits = (unsigned short)((got[q] >> (16 * e)) & 0xbfffu);
                            half_t yv = __builtin_bit_cast(half_t, bits);
                            if ((bits & 0x7fffu) == kDecNanCode) yv = __builtin_bit_cast(half_t, (unsigned short)0x7e00u);
                            nv[e] = ly.residual ? (half_t)((float)yv + (float)old[e]) : yv;
                        }
                        *reinterpret_cast<half4_t*>(&in_vec[(k + 1) & 1][blk * 4]) = nv;
                    }
                }
                dec_barrier();  // B3: the next input is in LDS
                if (k == 0) {
                    // With every block's entry seen here, every block is past its reads of h_prev and c_prev, which hn / cn may
                    // be.  Without (a wait gave up, the entries were made here), nobody knows that: the new state is parked.
                    parked = parked_lds != 0u;
                    if (owner) {
                        (parked ? p.parked_h : ly.hn)[pj] = keep_h;
                        (parked ? p.parked_c : ly.cn)[pj] = keep_c;
                    }
                }
                if (k == 0 && pw == kDecPollWaves - 1) {
                    // The look for parked state may come any time after this block's own note (a device-scope store, before the
                    // polls that have just ended) has arrived: here the answer travels while the next layer is at work.
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    parked_seen = __hip_atomic_load(parked_any, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (k == kLastExchange && pw == kDecPollWaves - 1) {
                    if (parked_seen == g) store_parked();
                    if (lane == 0) __hip_atomic_store(my_notes, g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        if (kLastExchange >= 0 && parked && pw == 0) {
            __threadfence();  // the parked state is in place
            if (lane == 0) {
                __hip_atomic_store(parked_any, g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(my_notes + 2, g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            store_parked();
        }
    }
}

}  // namespace pimhip
