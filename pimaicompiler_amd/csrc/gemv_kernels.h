// fp16 batch-1 GEMV kernels for gfx950 (fp16 storage, fp32 accumulation, one rounding at the store).
//
// Two weight orders exist on this path, named after the operand order of the product:
//   MV ("W_X_I"): y[out] = W[out,in] . x[in]   -- weight rows contiguous along the reduction
//   VM ("I_X_W"): y[out] = x[in] . A[in,out]   -- weight rows contiguous along the outputs
// plus VV, the dot product of two vectors.  Every kernel takes the fused epilogue
// y = act(acc + bias) that the reference's addmv kernels define
// (runtime/include/executor/op_executor/custom_ops.h:216-381: bias added after the alpha/beta
// combination, ReLU applied last).
//
// All of them are HBM-bound: each weight element is read from memory exactly once per launch
// through 16-byte non-temporal loads, x stays cache resident, and the only cross-lane traffic is
// the final reduction.
#pragma once

#include "device_common.h"

namespace pimhip
{
// ---------------------------------------------------------------------------------------------
// MV order, vector path.  Requirements checked by the launcher: K % 8 == 0, ldw % 8 == 0,
// W / x 16-byte aligned.
//
// A block holds WAVES wavefronts.  KS consecutive wavefronts share one group of R rows and split
// the reduction dimension between them in an interleaved fashion (wave ks takes 16-byte chunks
// ks*64 + lane, then strides by 64*KS), so one block covers (WAVES / KS) * R rows.  Each lane
// keeps U chunks per row in flight: R*U independent 16-byte weight loads per lane per iteration.
// ---------------------------------------------------------------------------------------------
// SPLIT: x is the concatenation of two vectors that lie apart (x: the first split_chunks 16-byte pieces, x2: the rest);
// compiled out of every other instance.  KEEP: the weight is read with plain loads (load_weight).
template <int R, int U, int WAVES, int KS, bool SPLIT = false, bool KEEP = false>
__device__ __forceinline__ void gemv_mv_f16_body(const half_t* __restrict__ W, const half_t* __restrict__ x,
                                                 const half_t* __restrict__ bias, half_t* __restrict__ y, int N,
                                                 int K, long ldw, int relu, int block,
                                                 const half_t* __restrict__ x2 = nullptr, int split_chunks = 0)
{
    static_assert(WAVES % KS == 0, "KS must divide WAVES");
    constexpr int RG = WAVES / KS;  // row groups per block
    __shared__ float red[WAVES][R];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int rg = wave / KS;
    const int ks = wave % KS;
    const long row0 = ((long)block * RG + rg) * R;

    float acc[R];
    const half8_t* wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        acc[r] = 0.0f;
        long row = row0 + r;
        if (row > N - 1) row = N - 1;  // out-of-range rows re-read the last row and are never stored
        wrow[r] = reinterpret_cast<const half8_t*>(W + row * ldw);
    }
    const half8_t* xv = reinterpret_cast<const half8_t*>(x);
    const half8_t* xv2 = SPLIT ? reinterpret_cast<const half8_t*>(x2) - split_chunks : nullptr;  // (indexed from split_chunks on)
    auto x_at = [&](int c) { return (SPLIT && c >= split_chunks) ? xv2[c] : xv[c]; };
    const int nchunks = K >> 3;
    constexpr int STEP = 64 * KS;

    int c = ks * 64 + lane;
    // Main loop: U chunks per row in flight, all of them in range.
    for (; c + (U - 1) * STEP < nchunks; c += U * STEP) {
        half8_t xr[U];
        half8_t wr[R][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int r = 0; r < R; ++r) wr[r][u] = load_weight<KEEP>(wrow[r] + c + u * STEP);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) xr[u] = x_at(c + u * STEP);
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = dot8(wr[r][u], xr[u], acc[r]);
        }
    }
    // Tail: one chunk per row at a time.
    for (; c < nchunks; c += STEP) {
        half8_t wr[R];
#pragma unroll
        for (int r = 0; r < R; ++r) wr[r] = load_weight<KEEP>(wrow[r] + c);
        const half8_t xr = x_at(c);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = dot8(wr[r], xr, acc[r]);
    }

#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);

    if (KS > 1) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) red[wave][r] = acc[r];
        }
        __syncthreads();
        if (ks == 0 && lane < R) {
            float v = 0.0f;
#pragma unroll
            for (int s = 0; s < KS; ++s) v += red[rg * KS + s][lane];
            const long row = row0 + lane;
            if (row < N) {
                if (bias) v += (float)bias[row];
                if (relu) v = relu_f32(v);
                y[row] = (half_t)v;
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const long row = row0 + r;
            if (lane == r && row < N) {
                float v = acc[r];
                if (bias) v += (float)bias[row];
                if (relu) v = relu_f32(v);
                y[row] = (half_t)v;
            }
        }
    }
}

template <int R, int U, int WAVES, int KS>
__global__ __launch_bounds__(WAVES * 64) void gemv_mv_f16_kernel(const half_t* __restrict__ W,
                                                                 const half_t* __restrict__ x,
                                                                 const half_t* __restrict__ bias,
                                                                 half_t* __restrict__ y, int N, int K, long ldw,
                                                                 int relu)
{
    gemv_mv_f16_body<R, U, WAVES, KS>(W, x, bias, y, N, K, ldw, relu, blockIdx.x);
}

// The same for a small matrix that is used again and again between other work: plain loads (load_weight).  A kernel of its
// own, chosen on the host, so that the streaming kernel stays as it is.
template <int R, int U, int WAVES, int KS>
__global__ __launch_bounds__(WAVES * 64) void gemv_mv_keep_f16_kernel(const half_t* __restrict__ W,
                                                                      const half_t* __restrict__ x,
                                                                      const half_t* __restrict__ bias,
                                                                      half_t* __restrict__ y, int N, int K, long ldw,
                                                                      int relu)
{
    gemv_mv_f16_body<R, U, WAVES, KS, false, true>(W, x, bias, y, N, K, ldw, relu, blockIdx.x);
}

// y = act(W . cat(x1, x2) + bias) without the concatenation: the second operand of the RNNT joint network's first layer
// is cat(encoder frame, prediction), which the reference either materialises or splits the product over
// (compiler/source/frontend/optimizer/remove_cat_for_addmm.cpp:46-191: two dependent launches).
template <int R, int U, int WAVES, int KS, bool KEEP>
__global__ __launch_bounds__(WAVES * 64) void gemv_mv_cat2_f16_kernel(const half_t* __restrict__ W,
                                                                      const half_t* __restrict__ x1,
                                                                      const half_t* __restrict__ x2, int split_chunks,
                                                                      const half_t* __restrict__ bias,
                                                                      half_t* __restrict__ y, int N, int K, long ldw,
                                                                      int relu)
{
    gemv_mv_f16_body<R, U, WAVES, KS, true, KEEP>(W, x1, bias, y, N, K, ldw, relu, blockIdx.x, x2, split_chunks);
}

// Several independent MV GEMVs in one launch (sibling projections that the reference issues on separate
// streams, runtime/source/executor/op_executor/stream_ops_executor.cpp:36-47).  Blocks
// [block_begin[i], block_begin[i+1]) work on problem i.
static constexpr int kGemvGroupMax = 32;
struct GemvGroupArgs {
    const half_t* W[kGemvGroupMax];
    const half_t* x[kGemvGroupMax];
    const half_t* bias[kGemvGroupMax];
    half_t* y[kGemvGroupMax];
    int N[kGemvGroupMax];
    int K[kGemvGroupMax];
    int relu[kGemvGroupMax];
    int block_begin[kGemvGroupMax + 1];
    int count;
};

// Each problem runs with the block shape a launch of its own would use for its row length (long rows: the four
// wavefronts of a block split the reduction of two rows; shorter rows: two wavefronts per pair of rows).
static constexpr int kGemvGroupThreads = 256;
static constexpr int kGemvGroupLongRow = 4096;
__host__ __device__ inline int gemv_group_rows_per_block(int K) { return K >= kGemvGroupLongRow ? 2 : 4; }

template <bool KEEP>  // the group's weights together are small: plain loads (load_weight)
__global__ __launch_bounds__(kGemvGroupThreads) void gemv_mv_f16_group_kernel(GemvGroupArgs g)
{
    int i = 0;
    while (i + 1 < g.count && (int)blockIdx.x >= g.block_begin[i + 1]) ++i;
    const int block = (int)blockIdx.x - g.block_begin[i];
    if (g.K[i] >= kGemvGroupLongRow)
        gemv_mv_f16_body<2, 4, 4, 4, false, KEEP>(g.W[i], g.x[i], g.bias[i], g.y[i], g.N[i], g.K[i], (long)g.K[i], g.relu[i], block);
    else
        gemv_mv_f16_body<2, 2, 4, 2, false, KEEP>(g.W[i], g.x[i], g.bias[i], g.y[i], g.N[i], g.K[i], (long)g.K[i], g.relu[i], block);
}

// MV order, any K / leading dimension / alignment: one wavefront per row, 2-byte loads.
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_mv_f16_generic_kernel(const half_t* __restrict__ W,
                                                                         const half_t* __restrict__ x,
                                                                         const half_t* __restrict__ bias,
                                                                         half_t* __restrict__ y, int N, int K,
                                                                         long ldw, int relu)
{
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * WAVES + (threadIdx.x >> 6);
    if (row >= N) return;
    const half_t* w = W + row * ldw;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) acc = fmaf((float)w[k], (float)x[k], acc);
    acc = wave_sum(acc);
    if (lane == 0) {
        if (bias) acc += (float)bias[row];
        if (relu) acc = relu_f32(acc);
        y[row] = (half_t)acc;
    }
}

// ---------------------------------------------------------------------------------------------
// VM order, vector path.  Requirements: N % 8 == 0, lda % 8 == 0, A 16-byte aligned.
//
// A block owns CW = 8 * LPR adjacent outputs and a slice [k_begin, k_end) of the reduction.  LPR lanes (8 columns,
// one 16-byte load each) cover the block's part of one weight row, so a wavefront reads 64 / LPR rows per load
// instruction and the block's wavefronts interleave over the rows of the slice, U loads in flight per lane.
// gridDim.y slices cover K.  With one slice the block finishes the outputs itself.  With several, the blocks of all
// slices but the last store their CW partial sums (fp32) as 32-byte records in `partial[slice][N]` and exit; the blocks
// of the LAST slice add the records to their own sums, in an order that depends on the slice index only (so the result
// is the same in every run), and apply the epilogue.
//
// A record that has not arrived yet holds kVmEmpty in every word (the bit pattern 0xffffffff: a NaN that no sum of
// products of fp16 values can be, since arithmetic yields the canonical NaN or the widened payload of an fp16 NaN), so
// the reducing block polls each record until none of its words is kVmEmpty, adds it and writes kVmEmpty back for the
// next launch.  Records travel with device-scope (sc1) stores and loads; there is no fence (a device-scope fence writes
// back and invalidates the XCD's whole L2, once per block) and no ticket counter (store, acknowledgement, atomic,
// loads would be three trips through the memory side after the last block's arithmetic; polling is one).
//
// What the scheme assumes of the dispatcher, and what it does not: the producers never wait for anything, so each of
// them finishes whatever else occupies the GPU, in any dispatch order; results never depend on the order.  That the
// reducing blocks seldom wait long does: workgroups are dealt to the eight XCDs round-robin by linear id and each
// XCD starts its share in that order, so within every XCD the producers (slices 0..last-1) are started before that
// XCD's reducing blocks (the last slice), and a reducing block on one XCD waits at most for the other XCDs to get
// through the producers dealt to them.  When other work holds CUs of one XCD (a resident sequence kernel on another
// stream) that wait grows by as much as that XCD is held up.  It is bounded all the same: after `spin_limit` polls
// of one record (none at all with a limit of 0, which is how a test forces the condition from the host), or one second,
// the lane gives up on the record and computes that slice's sums for its eight columns itself, with the producer's own
// order of operations, so the result has the bits it would have had.  The record may still arrive later and would then
// sit in the workspace as if it belonged to the next launch: the lane raises *poison (a device word the reducing blocks
// of every launch look at) and *status (for the host), and until the host has refilled the records and cleared both,
// reducing blocks do not look at records at all and compute every slice themselves: slow, but right.
// ---------------------------------------------------------------------------------------------
// Destinations of a VM product: the same result is stored to `count` buffers (the GNMT attention context goes
// straight into three concatenation buffers, runtime/source/executor/op_executor/aten_ops_executor.cpp:694-737).
static constexpr int kGemvMaxOuts = 4;
struct GemvOuts {
    half_t* y[kGemvMaxOuts];
    int count;
};

// 32 contiguous bytes written at device scope (partial sums cross CUs and XCDs).
__device__ __forceinline__ void store32_device_scope(float* p, const float (&v)[8])
{
    const float4_t lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\tglobal_store_dwordx4 %0, %2, off offset:16 sc1" : : "v"(p), "v"(lo), "v"(hi) : "memory");
}
// One 32-byte record of partial sums read at device scope (both halves issued together, one wait).
__device__ __forceinline__ void load32_device_scope_one(const float* p, float4_t& lo, float4_t& hi)
{
    asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(lo), "=&v"(hi)
                 : "v"(p)
                 : "memory");
}


template <int WAVES, int U, int LPR>
__global__ __launch_bounds__(WAVES * 64) void gemv_vm_f16_kernel(const half_t* __restrict__ x,
                                                                 const half_t* __restrict__ A,
                                                                 const half_t* __restrict__ bias,
                                                                 GemvOuts outs, int K, int N, long lda,
                                                                 int relu, int k_per_slice, float* partial,
                                                                 unsigned int* status, unsigned int* poison,
                                                                 unsigned int spin_limit)
{
    static_assert(LPR == 16 || LPR == 32 || LPR == 64, "lanes per weight row");
    constexpr int RPW = 64 / LPR;          // rows per wavefront and load instruction
    constexpr int GROUPS = WAVES * RPW;    // row groups per block = LDS rows of the reduction
    constexpr int STEP = GROUPS;           // rows between consecutive loads of one lane
    __shared__ float red[GROUPS][8][LPR];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int cg = lane % LPR;             // which 8 columns of the block
    const int grp = wave * RPW + lane / LPR;
    const long col0 = ((long)blockIdx.x * LPR + cg) * 8;
    const bool col_ok = col0 < N;
    const int k_begin = blockIdx.y * k_per_slice;
    const int k_end = min(K, k_begin + k_per_slice);

    // (asked for now by the blocks that will reduce, needed when they start to: it travels behind the block's own rows)
    unsigned int poisoned = 0u;
    if (gridDim.y > 1 && blockIdx.y == gridDim.y - 1) poisoned = __hip_atomic_load(poison, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;

    if (col_ok) {
        const half_t* a = A + col0;
        int k = k_begin + grp;
        for (; k + (U - 1) * STEP < k_end; k += U * STEP) {
            half8_t ar[U];
            float xr[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                ar[u] = load_stream(reinterpret_cast<const half8_t*>(a + (long)(k + u * STEP) * lda));
#pragma unroll
            for (int u = 0; u < U; ++u) xr[u] = (float)x[k + u * STEP];
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmaf((float)ar[u][j], xr[u], acc[j]);
            }
        }
        for (; k < k_end; k += STEP) {
            const half8_t ar = load_stream(reinterpret_cast<const half8_t*>(a + (long)k * lda));
            const float xr = (float)x[k];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf((float)ar[j], xr, acc[j]);
        }
    }

    // Combine the GROUPS partial sums of each column in LDS, in group order; lanes tid < LPR end up with the block's result.
#pragma unroll
    for (int j = 0; j < 8; ++j) red[grp][j][cg] = acc[j];
    __syncthreads();
    const bool finisher = tid < LPR && col_ok;  // tid < LPR: cg == tid, grp == 0
    if (tid < LPR) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = red[0][j][cg];
#pragma unroll
            for (int g = 1; g < GROUPS; ++g) v += red[g][j][cg];
            acc[j] = v;
        }
    }

    auto epilogue_store = [&](const float (&v)[8]) {
        half8_t out;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float r = v[j];
            if (bias) r += (float)bias[col0 + j];
            if (relu) r = relu_f32(r);
            out[j] = (half_t)r;
        }
        for (int o = 0; o < outs.count; ++o) *reinterpret_cast<half8_t*>(outs.y[o] + col0) = out;
    };

    const int nslices = gridDim.y;
    if (nslices == 1) {
        if (finisher) epilogue_store(acc);
        return;
    }

    const int last = nslices - 1;
    if ((int)blockIdx.y != last) {
        if (finisher) store32_device_scope(partial + (long)blockIdx.y * N + col0, acc);
        return;
    }
    float own[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        own[j] = acc[j];  // meaningful in the finisher lanes
        acc[j] = 0.0f;
    }
    // Row group g adds the records of slices g, g + GROUPS, ... < last in that order.
    if (col_ok) {
        for (int sl = grp; sl < last; sl += GROUPS) {
            float* rec = partial + (long)sl * N + col0;
            float4_t lo, hi;
            unsigned int spins = 0;
            unsigned long long t_first = 0ull;
            bool have = false;
            while (poisoned == 0u) {
                if (spins > 0u && (spins & 255u) == 0u && wait_clock_expired(spins, t_first)) spins = 0xffffffffu;  // gives up below
                if (spins++ >= spin_limit) {
                    __hip_atomic_store(poison, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    break;
                }
                load32_device_scope_one(rec, lo, hi);
                bool ok = true;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    ok = ok && __builtin_bit_cast(unsigned int, lo[j]) != kVmEmpty && __builtin_bit_cast(unsigned int, hi[j]) != kVmEmpty;
                if (ok) {
                    have = true;
                    break;
                }
            }
            if (have) {
                const float e = __builtin_bit_cast(float, kVmEmpty);
                const float empty[8] = {e, e, e, e, e, e, e, e};
                store32_device_scope(rec, empty);
            } else {
                // Slice sl's sums for these eight columns, as its own block makes them: every row group's rows in ascending
                // order, then the groups in order.
                const half_t* a = A + col0;
                const int ks_begin = sl * k_per_slice, ks_end = min(K, ks_begin + k_per_slice);
                float v[8];
                for (int g = 0; g < GROUPS; ++g) {
                    float part[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) part[j] = 0.0f;
                    for (int k = ks_begin + g; k < ks_end; k += STEP) {
                        const half8_t ar = *reinterpret_cast<const half8_t*>(a + (long)k * lda);
                        const float xr = (float)x[k];
#pragma unroll
                        for (int j = 0; j < 8; ++j) part[j] = fmaf((float)ar[j], xr, part[j]);
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = g == 0 ? part[j] : v[j] + part[j];
                }
                lo = float4_t{v[0], v[1], v[2], v[3]};
                hi = float4_t{v[4], v[5], v[6], v[7]};
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] += lo[j];
                acc[4 + j] += hi[j];
            }
        }
    }
    __syncthreads();  // the first lanes have read `red` above before it is written again
#pragma unroll
    for (int j = 0; j < 8; ++j) red[grp][j][cg] = acc[j];
    __syncthreads();
    if (finisher) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            v[j] = red[0][j][cg];
#pragma unroll
            for (int g = 1; g < GROUPS; ++g) v[j] += red[g][j][cg];
            v[j] += own[j];
        }
        epilogue_store(v);
    }
}

// VM order, any N / leading dimension / alignment: 2-byte loads.  A block of 16 wavefronts owns 64 adjacent output
// columns (one per lane); wavefront g takes the rows g, g + 16, ... and the sixteen partial sums meet in LDS.
static constexpr int kVmGenericWaves = 16;
__global__ __launch_bounds__(64 * kVmGenericWaves) void gemv_vm_f16_generic_kernel(const half_t* __restrict__ x,
                                                                                   const half_t* __restrict__ A,
                                                                                   const half_t* __restrict__ bias,
                                                                                   GemvOuts outs, int K, int N, long lda,
                                                                                   int relu)
{
    __shared__ float red[kVmGenericWaves][64];
    const int lane = threadIdx.x & 63;
    const int g = threadIdx.x >> 6;
    const long col = (long)blockIdx.x * 64 + lane;
    float acc = 0.0f;
    if (col < N) {
        int k = g;
        for (; k + 3 * kVmGenericWaves < K; k += 4 * kVmGenericWaves) {
            half_t a[4], xv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a[u] = A[(long)(k + u * kVmGenericWaves) * lda + col];
                xv[u] = x[k + u * kVmGenericWaves];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) acc = fmaf((float)a[u], (float)xv[u], acc);
        }
        for (; k < K; k += kVmGenericWaves) acc = fmaf((float)A[(long)k * lda + col], (float)x[k], acc);
    }
    red[g][lane] = acc;
    __syncthreads();
    if (g == 0 && col < N) {
        float v = red[0][lane];
#pragma unroll
        for (int w = 1; w < kVmGenericWaves; ++w) v += red[w][lane];
        if (bias) v += (float)bias[col];
        if (relu) v = relu_f32(v);
        for (int o = 0; o < outs.count; ++o) outs.y[o][col] = (half_t)v;
    }
}

// ---------------------------------------------------------------------------------------------
// C[m][n] = A[m][n] + B, B either [m][n] or one row [n] added to every row (the reference's custom_add,
// runtime/include/executor/op_executor/custom_ops.h:383-433).  The exact sum of two fp16 values rounded once to
// fp16, which is also what the reference's half2 addition yields.  C may alias A or B.  HBM-bound: 6 bytes per element.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void add_f16_vec_kernel(const half_t* A, const half_t* B, half_t* C, long total8,
                                                          long row8, int b_broadcast)
{
    // Units of 8 halves (16 bytes); row8 = n / 8.
    const long stride = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total8; i += stride) {
        const half8_t a = reinterpret_cast<const half8_t*>(A)[i];
        const half8_t b = reinterpret_cast<const half8_t*>(B)[b_broadcast ? (i % row8) : i];
        half8_t c;
#pragma unroll
        for (int e = 0; e < 8; ++e) c[e] = (half_t)((float)a[e] + (float)b[e]);
        reinterpret_cast<half8_t*>(C)[i] = c;
    }
}

__global__ __launch_bounds__(256) void add_f16_generic_kernel(const half_t* A, const half_t* B, half_t* C, long total,
                                                              long n, int b_broadcast)
{
    const long stride = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
        C[i] = (half_t)((float)A[i] + (float)B[b_broadcast ? (i % n) : i]);
}

// ---------------------------------------------------------------------------------------------
// Measurement aid: reads n16 16-byte pieces with the same streaming loads the GEMV kernels use and keeps nothing
// (the sum only exists so that the loads are not removed; `sink` is written if it equals an impossible value).  What
// a launch of this kernel takes is the floor for any kernel that has to read the same bytes once.
// ---------------------------------------------------------------------------------------------
typedef float float4_probe_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void stream_read_probe_kernel(const float4_probe_t* __restrict__ data, long n16, float* sink)
{
    constexpr int U = 8;
    float s = 0.0f;
    const long stride = (long)gridDim.x * 256 * U;
    for (long base = (long)blockIdx.x * 256 * U + threadIdx.x; base < n16; base += stride) {
        float4_probe_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(data + min(base + (long)u * 256, n16 - 1));
#pragma unroll
        for (int u = 0; u < U; ++u) s += v[u][0] + v[u][3];
    }
    if (s == 1234.5f && sink) sink[0] = s;
}

// ---------------------------------------------------------------------------------------------
// VV: y[0] = sum_k a[k] * b[k].  One block of 1024 lanes; any K and alignment.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void dot_f16_kernel(const half_t* __restrict__ a, const half_t* __restrict__ b,
                                                       half_t* __restrict__ y, long K)
{
    __shared__ float red[16];
    float acc = 0.0f;
    for (long k = threadIdx.x; k < K; k += 1024) acc = fmaf((float)a[k], (float)b[k], acc);
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < 16; ++w) v += red[w];
        y[0] = (half_t)v;
    }
}

}  // namespace pimhip
