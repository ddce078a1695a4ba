// Input projection of one LSTM layer over all time steps, on the gfx950 matrix cores:
//   out[T, N] (fp32) = x[T, K] (fp16) . w[N, K]^T (fp16) + bias[N] (fp32)
// with N = 4H gate rows and K the layer's input width.  Both operands are contiguous along K, which is
// the natural operand layout of v_mfma_f32_16x16x32_f16: lane l of a wavefront supplies 8 consecutive K
// values of row (l % 16), starting at K offset 8 * (l / 16), for A (x) and for B (w) alike, and
// receives out rows 4 * (l / 16) .. + 3 of column (l % 16).
//
// Grid (1-D): one block of 256 lanes per 16 * NT output columns and 64 time steps, 8 * ceil(column tiles / 8) * row
// blocks per projection.  Requirements checked by the launcher:
// K % 8 == 0, 16-byte aligned x and w, row pitches % 8 == 0.
#pragma once

#include "device_common.h"

namespace pimhip
{
// A fragment-shaped load straight from global memory (16 lanes on 16 different rows) makes the vector cache look up one
// line per lane, which caps a CU at about 16 bytes per clock (measured: ~35 GB/s per CU, whatever the unrolling).  So
// the operands go through LDS, which only serves as a layout converter: the block reads 128-column slabs of its 64 x rows
// and 16 * NT w rows with row-contiguous 16-byte loads (16 adjacent lanes = 256 contiguous bytes), keeps the next slab in
// registers while the current one is multiplied, and every wavefront reads its fragments from LDS with ds_read_b128 (row
// pitch 272 bytes: 16 lanes x 16 bytes fall into 64 distinct banks).  The four wavefronts split K inside a slab (one
// 32-wide MFMA step each) and each accumulates the whole 64 x 16 * NT tile; the four partial tiles are added through LDS
// in a fixed order at the end.
static constexpr int kXprojTile = 64;    // time steps per block
static constexpr int kXprojKSplit = 4;   // wavefronts per block = MFMA K steps per slab
static constexpr int kXprojSlab = 32 * kXprojKSplit;  // K values per slab (128)
static constexpr int kXprojPitch = kXprojSlab + 8;    // LDS row pitch in halves (272 bytes)

// Up to two projections of the same x in one launch (the two directions of a bidirectional layer): blocks
// [p * blocks_per_problem, (p + 1) * blocks_per_problem) work on weight / bias / output set p.
struct XprojProblems {
    const half_t* w[2];
    const float* bias[2];
    float* out[2];
    int blocks_per_problem;
};

// NT: column tiles of 16 per block (2, or 1 when a single row block would leave CUs without work).
template <int NT>
__global__ __launch_bounds__(256) void input_projection_f16_kernel(const half_t* __restrict__ x, XprojProblems problems,
                                                                  int T, int K, int N, long ldx, long ldw, int row_blocks)
{
    const int problem = blockIdx.x >= (unsigned)problems.blocks_per_problem ? 1 : 0;
    const int block = blockIdx.x - problem * problems.blocks_per_problem;
    const half_t* __restrict__ w = problems.w[problem];
    const float* __restrict__ bias = problems.bias[problem];
    float* __restrict__ out = problems.out[problem];
    constexpr int ROWS = kXprojTile + 16 * NT;            // LDS rows per slab: x rows first, then w rows
    constexpr int CHUNKS = ROWS * (kXprojSlab / 8);       // 16-byte pieces per slab
    constexpr int PER_LANE = CHUNKS / 256;                // 5, 6 or 8
    static_assert(CHUNKS % 256 == 0, "slab must divide evenly over the block");
    constexpr int SLAB_BYTES = ROWS * kXprojPitch * 2;
    constexpr int RED_BYTES = kXprojKSplit * 4 * NT * 64 * 16;
    constexpr int LDS_BYTES = 2 * SLAB_BYTES > RED_BYTES ? 2 * SLAB_BYTES : RED_BYTES;
    __shared__ __align__(16) unsigned char lds[LDS_BYTES];  // two slabs while multiplying, the partial tiles afterwards

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int ks = tid >> 6;  // this wavefront's MFMA step inside a slab
    const int r16 = lane & 15;
    const int kq = lane >> 4;  // which 8-wide K slice of a 32-wide MFMA step this lane feeds
    // Workgroups go to the eight XCDs round-robin by linear id, and each XCD has its own L2.  All row blocks of a column
    // tile are therefore given ids that are equal modulo 8: the tile's slice of w is then pulled into one L2 once and
    // shared by its row blocks, instead of crossing the fabric once per row block and XCD.
    const int xcd = block & 7;
    const int local = block >> 3;
    const int col_tile = (local / row_blocks) * 8 + xcd;
    if (col_tile * (16 * NT) >= N) return;  // whole block, before any barrier
    const int n_base = col_tile * (16 * NT);
    const int t_base = (local % row_blocks) * kXprojTile;

    // Global side of the slab copy: piece i of this lane is row (tid + 256 i) / 16, 8-wide column (tid + 256 i) % 16.
    const half_t* src[PER_LANE];
    int dst[PER_LANE];  // LDS offset in halves within a slab
    const int kcol = (tid & 15) * 8;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int row = (tid >> 4) + 16 * i;
        // rows past T or N duplicate the last row; their results are never stored
        src[i] = row < kXprojTile ? x + (long)min(t_base + row, T - 1) * ldx
                                  : w + (long)min(n_base + row - kXprojTile, N - 1) * ldw;
        dst[i] = row * kXprojPitch + kcol;
    }

    half8_t zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;
    float4_t acc[4][NT];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const int slabs = (K + kXprojSlab - 1) / kXprojSlab;
    // One register stage: the loads of slab s + 1 are issued before slab s is multiplied and written to the other LDS
    // buffer after it.  (A second register stage, with a barrier that does not wait for global loads, measured slower.)
    half8_t stage[PER_LANE];
    auto fetch = [&](int slab) {
        const int k = slab * kXprojSlab + kcol;
        const bool ok = k < K;  // K % 8 == 0: an 8-wide piece is entirely in or out of range
        const int kc = ok ? k : 0;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const half8_t v = *reinterpret_cast<const half8_t*>(src[i] + kc);
            stage[i] = ok ? v : zero;
        }
    };
    auto deposit = [&](int buf) {
        half_t* base = reinterpret_cast<half_t*>(lds + buf * SLAB_BYTES);
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) *reinterpret_cast<half8_t*>(base + dst[i]) = stage[i];
    };

    fetch(0);
    deposit(0);
    __syncthreads();
    for (int s = 0; s < slabs; ++s) {
        if (s + 1 < slabs) fetch(s + 1);
        const half_t* base = reinterpret_cast<const half_t*>(lds + (s & 1) * SLAB_BYTES) + ks * 32 + kq * 8;
        half8_t a[4], b[NT];
#pragma unroll
        for (int m = 0; m < 4; ++m) a[m] = *reinterpret_cast<const half8_t*>(base + (m * 16 + r16) * kXprojPitch);
#pragma unroll
        for (int n = 0; n < NT; ++n) b[n] = *reinterpret_cast<const half8_t*>(base + (kXprojTile + n * 16 + r16) * kXprojPitch);
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m], b[n], acc[m][n], 0, 0, 0);
        // Slab s + 1 goes into the other buffer, which every wavefront stopped reading before the previous barrier.
        if (s + 1 < slabs) deposit((s + 1) & 1);
        __syncthreads();
    }

    float(*red)[4 * NT][64][4] = reinterpret_cast<float(*)[4 * NT][64][4]>(lds);  // [K split][tile][lane][4 rows]
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) *reinterpret_cast<float4_t*>(&red[ks][m * NT + n][lane][0]) = acc[m][n];
    __syncthreads();

    // Wavefront `ks` now finishes the row tile m = ks: lane (r16, kq) holds rows 4 * kq .. + 3 of column r16 of a tile.
    const int m = ks;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        float4_t v = *reinterpret_cast<const float4_t*>(&red[0][m * NT + n][lane][0]);
#pragma unroll
        for (int q = 1; q < kXprojKSplit; ++q) {
            const float4_t p = *reinterpret_cast<const float4_t*>(&red[q][m * NT + n][lane][0]);
            v[0] += p[0];
            v[1] += p[1];
            v[2] += p[2];
            v[3] += p[3];
        }
        const int col = n_base + n * 16 + r16;
        if (col < N) {
            const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t_base + m * 16 + kq * 4 + i;
                if (t < T) out[(long)t * N + col] = v[i] + bv;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The same product with w re-laid out once (at plan creation) in MFMA fragment order, so that w never passes through
// LDS: a wavefront's B fragment of a (16-row tile j, 32-wide K step s) is the 1 KB at ((j * ksteps + s) * 64 + lane) * 8
// halves, lane = kq * 16 + r16 holding w[16 j + r16][32 s + 8 kq .. + 7]; rows past N and columns past K are zero;
// ksteps = padded K / 32 with K padded to a multiple of kXprojSlab.  Only x goes through LDS, which halves the LDS
// traffic per MFMA (the bound of the kernel above).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pack_w_fragments_kernel(const half_t* __restrict__ w, half_t* __restrict__ wp, int N, int K,
                                                               long ldw, int ntiles, int ksteps)
{
    const long chunk = (long)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece of the packed matrix
    const long total = (long)ntiles * ksteps * 64;
    if (chunk >= total) return;
    const int lane = (int)(chunk & 63);
    const long frag = chunk >> 6;
    const int s = (int)(frag % ksteps);
    const int j = (int)(frag / ksteps);
    const int row = j * 16 + (lane & 15);
    const int k = s * 32 + (lane >> 4) * 8;
    half8_t v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (half_t)0.0f;
    if (row < N && k < K) v = *reinterpret_cast<const half8_t*>(w + (long)row * ldw + k);  // K % 8 == 0
    reinterpret_cast<half8_t*>(wp)[chunk] = v;
}

struct XprojPackedProblems {
    const half_t* wp[2];
    const float* bias[2];
    float* out[2];
    int blocks_per_problem;
};

// Ranges of 16-byte words that the blocks behind the projection's own set to all-ones bytes: the hand-over slots of the
// pipeline launch that follows (lstm_xcd_kernels.h), marked "not written yet" beside the projection instead of by a launch
// of their own between the two.
struct XprojFill {
    unsigned int* ptr[6];
    unsigned int words16[6];
    int count;        // ranges; 0: the launch has no such blocks
    int first_block;  // the first block that fills
    int blocks;       // how many do
};

__device__ __forceinline__ void xproj_fill_ones(const XprojFill& f, int fb, int n_threads)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 ones = {~0u, ~0u, ~0u, ~0u};
    for (int r = 0; r < f.count; ++r) {
        u32x4* p = reinterpret_cast<u32x4*>(f.ptr[r]);
        const size_t n = f.words16[r];
        for (size_t i = (size_t)fb * n_threads + threadIdx.x; i < n; i += (size_t)f.blocks * n_threads) p[i] = ones;
    }
}

// KS wavefronts per block, one 32-wide K step of a (32 * KS)-wide slab each.
template <int NT, int KS = kXprojKSplit>
__global__ __launch_bounds__(64 * KS) void input_projection_packed_f16_kernel(const half_t* __restrict__ x, XprojPackedProblems problems,
                                                                         int T, int K, int N, long ldx, int ksteps,
                                                                         int row_blocks, XprojFill fill)
{
    if (fill.count > 0 && (int)blockIdx.x >= fill.first_block) {
        xproj_fill_ones(fill, (int)blockIdx.x - fill.first_block, 64 * KS);
        return;
    }
    constexpr int SLAB = 32 * KS;                          // K values per slab
    constexpr int PITCH = SLAB + 8;                        // LDS row pitch in halves
    constexpr int CPR = SLAB / 8;                          // 16-byte pieces per x row and slab
    constexpr int CHUNKS = kXprojTile * CPR;               // 16-byte pieces of an x slab
    constexpr int PER_LANE = CHUNKS / (64 * KS);           // 4
    constexpr int SLAB_BYTES = kXprojTile * PITCH * 2;
    constexpr int RED_BYTES = KS * 4 * NT * 64 * 16;
    constexpr int LDS_BYTES = 2 * SLAB_BYTES > RED_BYTES ? 2 * SLAB_BYTES : RED_BYTES;
    __shared__ __align__(16) unsigned char lds[LDS_BYTES];

    const int problem = blockIdx.x >= (unsigned)problems.blocks_per_problem ? 1 : 0;
    const int block = blockIdx.x - problem * problems.blocks_per_problem;
    const half_t* __restrict__ wp = problems.wp[problem];
    const float* __restrict__ bias = problems.bias[problem];
    float* __restrict__ out = problems.out[problem];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int ks = tid >> 6;
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int xcd = block & 7;  // column tiles pinned to one XCD, as above
    const int local = block >> 3;
    const int col_tile = (local / row_blocks) * 8 + xcd;
    if (col_tile * (16 * NT) >= N) return;
    const int n_base = col_tile * (16 * NT);
    const int t_base = (local % row_blocks) * kXprojTile;

    const half_t* src[PER_LANE];
    int dst[PER_LANE];
    const int kcol = (tid % CPR) * 8;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int row = tid / CPR + (64 * KS / CPR) * i;
        src[i] = x + (long)min(t_base + row, T - 1) * ldx;
        dst[i] = row * PITCH + kcol;
    }
    // This wavefront's B fragments: tile (col_tile * NT + n), K step 4 * slab + ks.
    const half8_t* wfrag[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) wfrag[n] = reinterpret_cast<const half8_t*>(wp) + ((long)(col_tile * NT + n) * ksteps + ks) * 64 + lane;

    half8_t zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (half_t)0.0f;
    float4_t acc[4][NT];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    const int slabs = (ksteps + KS - 1) / KS;
    half8_t stage[PER_LANE];
    half8_t b_next[NT];
    auto fetch = [&](int slab) {
        const int k = slab * SLAB + kcol;
        const bool ok = k < K;
        const int kc = ok ? k : 0;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const half8_t v = *reinterpret_cast<const half8_t*>(src[i] + kc);
            stage[i] = ok ? v : zero;
        }
#pragma unroll
        for (int n = 0; n < NT; ++n) b_next[n] = (slab * KS + ks < ksteps) ? wfrag[n][(long)slab * KS * 64] : zero;
    };
    auto deposit = [&](int buf) {
        half_t* base = reinterpret_cast<half_t*>(lds + buf * SLAB_BYTES);
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) *reinterpret_cast<half8_t*>(base + dst[i]) = stage[i];
    };

    fetch(0);
    deposit(0);
    __syncthreads();
    for (int s = 0; s < slabs; ++s) {
        half8_t b[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) b[n] = b_next[n];
        if (s + 1 < slabs) fetch(s + 1);
        const half_t* base = reinterpret_cast<const half_t*>(lds + (s & 1) * SLAB_BYTES) + ks * 32 + kq * 8;
        half8_t a[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) a[m] = *reinterpret_cast<const half8_t*>(base + (m * 16 + r16) * PITCH);
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m], b[n], acc[m][n], 0, 0, 0);
        if (s + 1 < slabs) deposit((s + 1) & 1);
        __syncthreads();
    }

    float(*red)[4 * NT][64][4] = reinterpret_cast<float(*)[4 * NT][64][4]>(lds);
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) *reinterpret_cast<float4_t*>(&red[ks][m * NT + n][lane][0]) = acc[m][n];
    __syncthreads();
    if (ks >= 4) return;  // four row tiles, finished by the first four wavefronts
    const int m = ks;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        float4_t v = *reinterpret_cast<const float4_t*>(&red[0][m * NT + n][lane][0]);
#pragma unroll
        for (int q = 1; q < KS; ++q) {
            const float4_t p = *reinterpret_cast<const float4_t*>(&red[q][m * NT + n][lane][0]);
            v[0] += p[0];
            v[1] += p[1];
            v[2] += p[2];
            v[3] += p[3];
        }
        const int col = n_base + n * 16 + r16;
        if (col < N) {
            const float bv = bias ? bias[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t_base + m * 16 + kq * 4 + i;
                if (t < T) out[(long)t * N + col] = v[i] + bv;
            }
        }
    }
}

// bsum[i] = b_ih[i] + b_hh[i] in fp32 (either may be null, meaning zero).
__global__ void lstm_bias_sum_kernel(const half_t* __restrict__ b_ih, const half_t* __restrict__ b_hh,
                                     float* __restrict__ bsum, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) bsum[i] = (b_ih ? (float)b_ih[i] : 0.0f) + (b_hh ? (float)b_hh[i] : 0.0f);
}

}  // namespace pimhip
