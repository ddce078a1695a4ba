// The input projection of the C ABI (include/pimhip.h): the one matrix-core kernel of the path, with plain and
// fragment-ordered weights, and the two small preparation kernels that live beside it.
#include "api_common.h"
#include "xproj_kernels.h"

using namespace pimhip;

namespace pimhip
{
int launch_input_projection(int count, float* const* out, const half_t* x, const half_t* const* w, const float* const* bias,
                            int64_t T, int64_t K, int64_t N, hipStream_t s, int64_t ldx, int64_t ldw)
{
    if (ldx == 0) ldx = K;
    if (ldw == 0) ldw = K;
    if (T <= 0 || N <= 0) return PIMHIP_OK;
    if (K % 8 != 0 || !aligned16(x))
        return fail(PIMHIP_ERR_UNSUPPORTED, "input projection needs in_w %% 8 == 0 (got %lld) and 16-byte aligned x and w", (long long)K);
    if (T > INT32_MAX || K > INT32_MAX || N > INT32_MAX) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "dimension above 2^31-1");
    XprojProblems pr;
    memset(&pr, 0, sizeof(pr));
    for (int p = 0; p < count; ++p) {
        if (!aligned16(w[p]))
            return fail(PIMHIP_ERR_UNSUPPORTED, "input projection needs in_w %% 8 == 0 (got %lld) and 16-byte aligned x and w", (long long)K);
        pr.w[p] = w[p];
        pr.bias[p] = bias[p];
        pr.out[p] = out[p];
    }
    // 64 time steps per block row.  Measured on MI355X for T = 50, 200, 800 and K = 240, 1024, 2048 (N = 4096): 32-column
    // tiles are fastest as soon as there are two row blocks, 16-column tiles with one (more blocks than CUs either way).
    const unsigned row_blocks = (unsigned)((T + kXprojTile - 1) / kXprojTile);
    auto blocks = [&](int cols) { return (unsigned)(((N + cols - 1) / cols + 7) / 8 * 8) * row_blocks; };
    if (row_blocks >= 2) {
        pr.blocks_per_problem = (int)blocks(32);
        input_projection_f16_kernel<2><<<blocks(32) * count, 256, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)ldx, (long)ldw, (int)row_blocks);
    } else {
        pr.blocks_per_problem = (int)blocks(16);
        input_projection_f16_kernel<1><<<blocks(16) * count, 256, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)ldx, (long)ldw, (int)row_blocks);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PIMHIP_ERR_HIP, "input projection launch failed: %s", hipGetErrorString(e));
    return PIMHIP_OK;
}

// The same with weights in fragment order (pack_w_fragments_kernel); N, K checked by the caller (plan creation).
int launch_input_projection_packed(int count, float* const* out, const half_t* x, const half_t* const* wp, const float* const* bias,
                                   int64_t T, int64_t K, int64_t N, int ksteps, hipStream_t s, const FillSegments* ones, int n_ones)
{
    if (T <= 0 || N <= 0) {
        if (ones && n_ones > 0) launch_fill_segments(*ones, n_ones, 0xffffffffu, s);
        return PIMHIP_OK;
    }
    // ranges to set to all-ones bytes beside the projection (whole 16-byte words, or a launch of their own does it)
    XprojFill fill;
    memset(&fill, 0, sizeof(fill));
    bool fill_here = ones && n_ones > 0 && n_ones <= 6;
    for (int r = 0; fill_here && r < n_ones; ++r)
        fill_here = (reinterpret_cast<uintptr_t>(ones->ptr[r]) & 15u) == 0 && (ones->words[r] & 3u) == 0 && ones->words[r] / 4 <= 0xffffffffull;
    if (ones && n_ones > 0 && !fill_here) launch_fill_segments(*ones, n_ones, 0xffffffffu, s);
    if (fill_here) {
        for (int r = 0; r < n_ones; ++r) {
            fill.ptr[r] = ones->ptr[r];
            fill.words16[r] = (unsigned int)(ones->words[r] / 4);
        }
        fill.count = n_ones;
        fill.blocks = 128;
    }
    XprojPackedProblems pr;
    memset(&pr, 0, sizeof(pr));
    for (int p = 0; p < count; ++p) {
        pr.wp[p] = wp[p];
        pr.bias[p] = bias[p];
        pr.out[p] = out[p];
    }
    const unsigned row_blocks = (unsigned)((T + kXprojTile - 1) / kXprojTile);
    auto blocks = [&](int cols) { return (unsigned)(((N + cols - 1) / cols + 7) / 8 * 8) * row_blocks; };
    // the projection's blocks first, the filling blocks behind them
    auto launch_as = [&](unsigned proj_blocks, auto launch) {
        fill.first_block = (int)proj_blocks;
        launch(proj_blocks + (unsigned)(fill.count > 0 ? fill.blocks : 0));
    };
    // Measured on MI355X (T = 50, 200, 800; K = 240, 1024, 2048; N = 4096): with one row block 16-column tiles and
    // eight wavefronts splitting K; with more, 32-column tiles, and eight wavefronts only for long rows and few row blocks.
    if (row_blocks >= 2) {
        pr.blocks_per_problem = (int)blocks(32);
        if (row_blocks <= 4 && K >= 2048)
            launch_as(blocks(32) * count, [&](unsigned grid) {
                input_projection_packed_f16_kernel<2, 8><<<grid, 512, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks, fill);
            });
        else
            launch_as(blocks(32) * count, [&](unsigned grid) {
                input_projection_packed_f16_kernel<2, 4><<<grid, 256, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks, fill);
            });
    } else {
        pr.blocks_per_problem = (int)blocks(16);
        launch_as(blocks(16) * count, [&](unsigned grid) {
            input_projection_packed_f16_kernel<1, 8><<<grid, 512, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks, fill);
        });
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PIMHIP_ERR_HIP, "input projection launch failed: %s", hipGetErrorString(e));
    return PIMHIP_OK;
}

void packed_geometry(int64_t in_w, int64_t n_out, int* ntiles, int* ksteps)
{
    *ksteps = (int)((in_w + kXprojSlab - 1) / kXprojSlab * kXprojSlab / 32);
    *ntiles = (int)((n_out + 63) / 64 * 4);
}

void launch_pack_w_fragments(const half_t* w, half_t* packed, int64_t n_out, int64_t in_w, int ntiles, int ksteps, hipStream_t s)
{
    const size_t chunks = (size_t)ntiles * ksteps * 64;
    pack_w_fragments_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, s>>>(w, packed, (int)n_out, (int)in_w, (long)in_w, ntiles, ksteps);
}

void launch_lstm_bias_sum(const half_t* b_ih, const half_t* b_hh, float* bsum, int n, hipStream_t s)
{
    lstm_bias_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(b_ih, b_hh, bsum, n);
}
}  // namespace pimhip

extern "C" int pimhip_input_projection(void* out, const void* x, const void* w, const void* bias, int64_t seq_len,
                                       int64_t in_w, int64_t n_out, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !x || !w) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, x and w must be non-null");
    if (seq_len < 0 || in_w < 0 || n_out < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "negative dimension");
    float* outs[1] = {(float*)out};
    const half_t* ws[1] = {(const half_t*)w};
    const float* bs[1] = {(const float*)bias};
    return launch_input_projection(1, outs, (const half_t*)x, ws, bs, seq_len, in_w, n_out, static_cast<hipStream_t>(stream), 0, 0);
}

extern "C" int pimhip_projection_packed_bytes(int64_t in_w, int64_t n_out, uint64_t* bytes)
{
    if (!bytes) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "bytes is null");
    if (in_w < 1 || n_out < 1 || in_w > INT32_MAX || n_out > INT32_MAX) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in_w=%lld n_out=%lld out of range", (long long)in_w, (long long)n_out);
    int ntiles = 0, ksteps = 0;
    packed_geometry(in_w, n_out, &ntiles, &ksteps);
    *bytes = (uint64_t)ntiles * (uint64_t)ksteps * 64u * 16u;
    return PIMHIP_OK;
}

extern "C" int pimhip_pack_projection_weight(void* packed, const void* w, int64_t in_w, int64_t n_out, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!packed || !w) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "packed and w must be non-null");
    if (in_w < 1 || n_out < 1 || in_w > INT32_MAX || n_out > INT32_MAX) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in_w=%lld n_out=%lld out of range", (long long)in_w, (long long)n_out);
    if (in_w % 8 != 0 || !aligned16(w) || !aligned16(packed))
        return fail(PIMHIP_ERR_UNSUPPORTED, "packing needs in_w %% 8 == 0 (got %lld) and 16-byte aligned pointers", (long long)in_w);
    int ntiles = 0, ksteps = 0;
    packed_geometry(in_w, n_out, &ntiles, &ksteps);
    launch_pack_w_fragments((const half_t*)w, (half_t*)packed, n_out, in_w, ntiles, ksteps, static_cast<hipStream_t>(stream));
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_input_projection_packed(void* out, const void* x, const void* packed, const void* bias, int64_t seq_len,
                                              int64_t in_w, int64_t n_out, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (seq_len < 0 || in_w < 1 || n_out < 1 || seq_len > INT32_MAX || in_w > INT32_MAX || n_out > INT32_MAX)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "seq_len=%lld in_w=%lld n_out=%lld out of range", (long long)seq_len, (long long)in_w, (long long)n_out);
    if (seq_len == 0) return PIMHIP_OK;
    if (!out || !x || !packed) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, x and packed must be non-null");
    if (in_w % 8 != 0 || !aligned16(x) || !aligned16(packed))
        return fail(PIMHIP_ERR_UNSUPPORTED, "input projection needs in_w %% 8 == 0 (got %lld) and 16-byte aligned x and packed", (long long)in_w);
    int ntiles = 0, ksteps = 0;
    packed_geometry(in_w, n_out, &ntiles, &ksteps);
    float* outs[1] = {(float*)out};
    const half_t* wps[1] = {(const half_t*)packed};
    const float* bs[1] = {(const float*)bias};
    return launch_input_projection_packed(1, outs, (const half_t*)x, wps, bs, seq_len, in_w, n_out, ksteps, static_cast<hipStream_t>(stream));
}
