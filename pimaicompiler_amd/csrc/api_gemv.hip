// The fp16 GEMV family of the C ABI (include/pimhip.h): both operand orders, the product over two vectors that lie apart,
// the grouped launch, bmm, add, dot, and the read-only probe the benchmark times beside them.
#include "api_common.h"
#include "../../include/pimhip_probe.h"
#include "gemv_kernels.h"

using namespace pimhip;

namespace
{
constexpr size_t kStaticScratchFloats = 64 * 1024;  // the array itself is in api_core.hip, where its address is looked up

int get_split_workspace(DeviceState* st, hipStream_t stream, size_t partial_elems, SplitWorkspace** out)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    SplitWorkspace& ws = st->workspaces[stream];
    const bool gave_up = ws.status && *ws.status != 0u;
    bool capturing = false;
    if (!ws.status || ws.partial_elems < partial_elems || gave_up) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
        capturing = capture != hipStreamCaptureStatusNone;
        // Allocation, synchronisation and the memset below are not for a graph.
        if (capturing && (!ws.status || ws.partial_elems < partial_elems))
            return fail(PIMHIP_ERR_UNSUPPORTED, "this I_X_W product needs its stream's workspace (re)allocated, which a graph must not "
                                                "record: run it once on this stream before the capture");
    }
    if (!ws.status) {
        PIMHIP_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&ws.status), sizeof(unsigned int), hipHostMallocMapped));
        *ws.status = 0u;
        PIMHIP_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&ws.status_dev), ws.status, 0));
        PIMHIP_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&ws.poison), sizeof(unsigned int)));
        PIMHIP_HIP_CHECK(hipMemsetAsync(ws.poison, 0, sizeof(unsigned int), stream));
    }
    // A reducing block of an earlier product on this stream gave up on a record.  That product's result was completed by
    // the block itself, and the products since have ignored the records (the poison word is up); outside a capture the
    // records are refilled here and both words cleared.  (Inside one the launch goes ahead as it is: right, only slower.)
    const bool recover = gave_up && !capturing;
    if (ws.partial_elems < partial_elems || recover) {
        // Work already queued on this stream may still use the old buffer.
        PIMHIP_HIP_CHECK(hipStreamSynchronize(stream));
        if (ws.partial_elems < partial_elems) {
            if (ws.partial) PIMHIP_HIP_CHECK(hipFree(ws.partial));
            ws.partial = nullptr;
            ws.partial_elems = 0;
            PIMHIP_HIP_CHECK(hipMalloc(&ws.partial, partial_elems * sizeof(float)));
            ws.partial_elems = partial_elems;
        }
        PIMHIP_HIP_CHECK(hipMemsetAsync(ws.partial, 0xff, ws.partial_elems * sizeof(float), stream));  // every word kVmEmpty
        PIMHIP_HIP_CHECK(hipMemsetAsync(ws.poison, 0, sizeof(unsigned int), stream));
        if (recover) ++ws.gave_up_events;
        *ws.status = 0u;
    }
    *out = &ws;
    return PIMHIP_OK;
}

// ---- GEMV launch selection ---------------------------------------------------------------------
template <int R, int U, int WAVES, int KS>
void launch_mv(const half_t* W, const half_t* x, const half_t* b, half_t* y, int N, int K, long ldw, int relu,
               hipStream_t s)
{
    constexpr int rows_per_block = (WAVES / KS) * R;
    const int grid = (N + rows_per_block - 1) / rows_per_block;
    // a small matrix is read with plain loads: its rows are still cached when its turn comes again (load_weight)
    const int keep = (unsigned long long)N * (unsigned long long)K * sizeof(half_t) <= kKeepCachedBytes;
    if (keep)
        gemv_mv_keep_f16_kernel<R, U, WAVES, KS><<<grid, WAVES * 64, 0, s>>>(W, x, b, y, N, K, ldw, relu);
    else
        gemv_mv_f16_kernel<R, U, WAVES, KS><<<grid, WAVES * 64, 0, s>>>(W, x, b, y, N, K, ldw, relu);
}

int gemv_mv(const half_t* W, const half_t* x, const half_t* bias, half_t* y, int64_t N, int64_t K, int64_t ldw,
            int relu, hipStream_t s)
{
    const bool vec_ok = (K % 8 == 0) && (ldw % 8 == 0) && aligned16(W) && aligned16(x);
    if (!vec_ok) {
        const int grid = (int)((N + 3) / 4);
        gemv_mv_f16_generic_kernel<4><<<grid, 256, 0, s>>>(W, x, bias, y, (int)N, (int)K, (long)ldw, relu);
        return PIMHIP_OK;
    }
    // Measured on MI355X over the (out, in) shapes of the GEMV sweep: long rows want the reduction split
    // over the four wavefronts of a block (more rows of the matrix open at once per CU would thrash DRAM
    // pages), short rows want two rows per wavefront.  Few rows: one row per block so that enough blocks exist.
    if (N < 1024) {
        if (K >= 2048)
            launch_mv<1, 4, 4, 4>(W, x, bias, y, (int)N, (int)K, (long)ldw, relu, s);
        else
            launch_mv<1, 2, 4, 4>(W, x, bias, y, (int)N, (int)K, (long)ldw, relu, s);
    } else if (K >= 4096) {
        launch_mv<2, 4, 4, 4>(W, x, bias, y, (int)N, (int)K, (long)ldw, relu, s);
    } else {
        launch_mv<2, 2, 4, 2>(W, x, bias, y, (int)N, (int)K, (long)ldw, relu, s);
    }
    return PIMHIP_OK;
}


// The records of the static scratch array instead of the stream's workspace: nothing is allocated, freed or
// synchronised (pimhip_execute_gemv_static).
int get_static_workspace(DeviceState* st, hipStream_t stream, size_t partial_elems, float** partial, unsigned int** status,
                         unsigned int** poison)
{
    if (!st->static_partial || !st->static_status || !st->static_poison)
        return fail(PIMHIP_ERR_NOT_INITIALIZED, "the static scratch buffer of this device has not been set up");
    if (partial_elems > kStaticScratchFloats)
        return fail(PIMHIP_ERR_UNSUPPORTED, "this I_X_W product needs %zu partial sums, the static scratch buffer holds %zu: "
                                            "use pimhip_execute_gemv", partial_elems, kStaticScratchFloats);
    if (*st->static_status != 0u) {
        // A reducing block of an earlier launch gave up on a record: that product was completed by the block itself, and
        // the launches since have ignored the records.  Outside a capture every word is brought back to kVmEmpty here with
        // fill kernels on this stream and both words are cleared (the status word first: the launch that set it has ended
        // once the stream has drained).  Inside a capture the launch goes ahead as it is: right, only slower.
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
        if (capture == hipStreamCaptureStatusNone) {
            PIMHIP_HIP_CHECK(hipStreamSynchronize(stream));
            *st->static_status = 0u;
            ++st->static_gave_up_events;
            launch_fill_u32(reinterpret_cast<unsigned int*>(st->static_partial), kStaticScratchFloats, kVmEmpty, stream);
            launch_fill_u32(st->static_poison, 1, 0u, stream);
            PIMHIP_HIP_CHECK(hipGetLastError());
        }
    }
    *partial = st->static_partial;
    *status = st->static_status_dev;
    *poison = st->static_poison;
    return PIMHIP_OK;
}

int gemv_vm(DeviceState* st, const half_t* x, const half_t* A, const half_t* bias, const GemvOuts& outs, int64_t K,
            int64_t N, int64_t lda, int relu, hipStream_t s, bool static_ws = false)
{
    bool vec_ok = (N % 8 == 0) && (lda % 8 == 0) && aligned16(A);
    for (int o = 0; o < outs.count; ++o) vec_ok = vec_ok && aligned16(outs.y[o]);
    if (!vec_ok) {
        const int grid = (int)((N + 63) / 64);
        gemv_vm_f16_generic_kernel<<<grid, 64 * kVmGenericWaves, 0, s>>>(x, A, bias, outs, (int)K, (int)N, (long)lda, relu);
        return PIMHIP_OK;
    }
    // Measured on MI355X: 128-column blocks (16 lanes per weight row, 4 rows per wavefront and load) with 8 loads in
    // flight per lane are fastest for every shape tried; a cross-block reduction costs 1 to 2 us, so K is sliced
    // only as far as needed for roughly one block per CU (64 blocks for a weight of a few MB), and not at all for
    // weights of up to 256 KB.
    constexpr int WAVES = 4, U = 8, LPR = 16;
    constexpr int GROUPS = WAVES * (64 / LPR);
    const int col_blocks = (int)((N + LPR * 8 - 1) / (LPR * 8));
    const int64_t weight_bytes = K * N * (int64_t)sizeof(half_t);
    int64_t target = weight_bytes / 65536;
    if (target < 64) target = 64;
    if (target > st->num_cus) target = st->num_cus;
    int slices = (int)((target + col_blocks / 2) / col_blocks);  // rounded: 250 column blocks on 256 CUs are not sliced
    const int max_slices = (int)((K + 31) / 32);
    if (slices > max_slices) slices = max_slices;
    if (weight_bytes <= 256 * 1024) slices = 1;
    if (slices < 1) slices = 1;
    int k_per_slice = (int)((K + slices - 1) / slices);
    k_per_slice = (k_per_slice + GROUPS - 1) / GROUPS * GROUPS;
    if (k_per_slice < GROUPS) k_per_slice = GROUPS;  // K == 0: one empty slice, y = act(bias)
    slices = (int)((K + k_per_slice - 1) / k_per_slice);
    if (slices < 1) slices = 1;
    float* partial = nullptr;
    unsigned int* status = nullptr;
    unsigned int* poison = nullptr;
    if (slices > 1) {
        // Records of all slices but the last: partial[slice][N].
        const size_t partial_elems = (size_t)(slices - 1) * (size_t)N;
        int rc;
        if (static_ws) {
            rc = get_static_workspace(st, s, partial_elems, &partial, &status, &poison);
        } else {
            SplitWorkspace* ws = nullptr;
            rc = get_split_workspace(st, s, partial_elems, &ws);
            if (rc == PIMHIP_OK) {
                partial = ws->partial;
                status = ws->status_dev;
                poison = ws->poison;
            }
        }
        if (rc != PIMHIP_OK) return rc;
    }
    dim3 grid(col_blocks, slices);
    gemv_vm_f16_kernel<WAVES, U, LPR><<<grid, WAVES * 64, 0, s>>>(x, A, bias, outs, (int)K, (int)N, (long)lda, relu,
                                                                    k_per_slice, partial, status, poison, st->vm_spin_limit);
    return PIMHIP_OK;
}

}  // namespace

namespace pimhip
{
void launch_add_f16_vec(const half_t* a, const half_t* b, half_t* c, long total8, long n8, int b_broadcast, int num_cus, hipStream_t s)
{
    // About 8 blocks per CU, each lane 16 bytes per operand and trip.
    long grid = (total8 + 255) / 256;
    if (grid > 8L * num_cus) grid = 8L * num_cus;
    add_f16_vec_kernel<<<(unsigned)grid, 256, 0, s>>>(a, b, c, total8, n8, b_broadcast);
}
}  // namespace pimhip

// ================================================================================================
// GEMV family
// ================================================================================================
namespace
{
int execute_gemv(void* out, const void* in, const void* weight, const void* bias, int64_t in_w, int64_t out_w,
                 int64_t ld_weight, int act, int order, void* stream, bool static_ws)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !in || !weight) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, in and weight must be non-null");
    if (in_w < 0 || out_w < 0 || in_w > INT32_MAX || out_w > INT32_MAX)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in_w=%lld out_w=%lld out of range", (long long)in_w, (long long)out_w);
    if (act != PIMHIP_ACT_NONE && act != PIMHIP_ACT_RELU) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown activation %d", act);
    if (order != PIMHIP_I_X_W && order != PIMHIP_W_X_I) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown operand order %d", order);
    if (out_w == 0) return PIMHIP_OK;
    const int64_t dense = (order == PIMHIP_W_X_I) ? in_w : out_w;
    if (ld_weight == 0) ld_weight = dense;
    if (ld_weight < dense)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ld_weight=%lld is below the row length %lld", (long long)ld_weight, (long long)dense);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int relu = act == PIMHIP_ACT_RELU;
    if (order == PIMHIP_W_X_I)
        rc = gemv_mv((const half_t*)weight, (const half_t*)in, (const half_t*)bias, (half_t*)out, out_w, in_w, ld_weight, relu, s);
    else {
        GemvOuts outs;
        memset(&outs, 0, sizeof(outs));
        outs.y[0] = (half_t*)out;
        outs.count = 1;
        rc = gemv_vm(st, (const half_t*)in, (const half_t*)weight, (const half_t*)bias, outs, in_w, out_w, ld_weight, relu, s, static_ws);
    }
    if (rc != PIMHIP_OK) return rc;
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}
}  // namespace

extern "C" int pimhip_execute_gemv(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                                   int64_t out_w, int64_t ld_weight, int act, int order, void* stream)
{
    return execute_gemv(out, in, weight, bias, in_w, out_w, ld_weight, act, order, stream, false);
}

extern "C" int pimhip_execute_gemv_cat2(void* out, const void* in1, int64_t in1_w, const void* in2, int64_t in2_w,
                                        const void* weight, const void* bias, int64_t out_w, int64_t ld_weight, int act,
                                        void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !in1 || !in2 || !weight) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, in1, in2 and weight must be non-null");
    if (in1_w < 1 || in2_w < 1 || out_w < 1) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in1_w=%lld in2_w=%lld out_w=%lld must be positive",
                                                         (long long)in1_w, (long long)in2_w, (long long)out_w);
    if (act != PIMHIP_ACT_NONE && act != PIMHIP_ACT_RELU) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "act=%d", act);
    const int64_t K = in1_w + in2_w;
    const int64_t ldw = ld_weight > 0 ? ld_weight : K;
    if (ldw < K) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ld_weight=%lld is less than in1_w + in2_w=%lld", (long long)ldw, (long long)K);
    if ((in1_w & 7) || (in2_w & 7) || (ldw & 7) || !aligned16(in1) || !aligned16(in2) || !aligned16(weight))
        return fail(PIMHIP_ERR_UNSUPPORTED, "both widths and the row pitch must be multiples of 8 and in1, in2, weight 16-byte aligned: "
                                            "concatenate and call pimhip_execute_gemv otherwise");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int relu = act == PIMHIP_ACT_RELU;
    const int N = (int)out_w;
    const int split = (int)(in1_w >> 3);
    const int keep = (unsigned long long)out_w * (unsigned long long)K * sizeof(half_t) <= kKeepCachedBytes;
    // (the launch shapes of gemv_mv)
    auto launch = [&](auto kernel, unsigned grid) {
        kernel<<<grid, 256, 0, s>>>((const half_t*)weight, (const half_t*)in1, (const half_t*)in2, split, (const half_t*)bias, (half_t*)out, N,
                                    (int)K, (long)ldw, relu);
    };
    if (out_w < 1024) {
        if (K >= 2048)
            keep ? launch(gemv_mv_cat2_f16_kernel<1, 4, 4, 4, true>, (unsigned)N) : launch(gemv_mv_cat2_f16_kernel<1, 4, 4, 4, false>, (unsigned)N);
        else
            keep ? launch(gemv_mv_cat2_f16_kernel<1, 2, 4, 4, true>, (unsigned)N) : launch(gemv_mv_cat2_f16_kernel<1, 2, 4, 4, false>, (unsigned)N);
    } else if (K >= 4096) {
        keep ? launch(gemv_mv_cat2_f16_kernel<2, 4, 4, 4, true>, (unsigned)(N + 1) / 2) : launch(gemv_mv_cat2_f16_kernel<2, 4, 4, 4, false>, (unsigned)(N + 1) / 2);
    } else {
        keep ? launch(gemv_mv_cat2_f16_kernel<2, 2, 4, 2, true>, (unsigned)(N + 3) / 4) : launch(gemv_mv_cat2_f16_kernel<2, 2, 4, 2, false>, (unsigned)(N + 3) / 4);
    }
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_execute_gemv_static(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                                          int64_t out_w, int64_t ld_weight, int act, int order, void* stream)
{
    return execute_gemv(out, in, weight, bias, in_w, out_w, ld_weight, act, order, stream, true);
}

extern "C" int pimhip_gemv_status(void* stream, int* gave_up)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!gave_up) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "gave_up must be non-null");
    std::lock_guard<std::mutex> lock(g_mutex);
    int flags = 0;
    auto it = st->workspaces.find(static_cast<hipStream_t>(stream));
    if (it != st->workspaces.end() && it->second.status && *it->second.status != 0u) flags |= 1;
    if (st->static_status && *st->static_status != 0u) flags |= 2;
    *gave_up = flags;
    return PIMHIP_OK;
}

extern "C" int pimhip_gemv_fallbacks(void* stream, uint64_t* events)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!events) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "events must be non-null");
    std::lock_guard<std::mutex> lock(g_mutex);
    uint64_t n = st->static_gave_up_events + ((st->static_status && *st->static_status != 0u) ? 1u : 0u);
    auto it = st->workspaces.find(static_cast<hipStream_t>(stream));
    if (it != st->workspaces.end()) n += it->second.gave_up_events + ((it->second.status && *it->second.status != 0u) ? 1u : 0u);
    *events = n;
    return PIMHIP_OK;
}

extern "C" int pimhip_set_gemv_spin_limit(unsigned int spin_limit)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    std::lock_guard<std::mutex> lock(g_mutex);
    st->vm_spin_limit = spin_limit;
    return PIMHIP_OK;
}

extern "C" int pimhip_execute_bmm(void* const* outs, int n_outs, const void* x, const void* A, int64_t k, int64_t n,
                                  void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!outs || !x || !A) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "outs, x and A must be non-null");
    if (n_outs < 1 || n_outs > kGemvMaxOuts) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "n_outs=%d not in [1, %d]", n_outs, kGemvMaxOuts);
    if (k < 0 || n < 0 || k > INT32_MAX || n > INT32_MAX) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "k=%lld n=%lld out of range", (long long)k, (long long)n);
    GemvOuts o;
    memset(&o, 0, sizeof(o));
    for (int i = 0; i < n_outs; ++i) {
        if (!outs[i]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "outs[%d] is null", i);
        o.y[i] = (half_t*)outs[i];
    }
    o.count = n_outs;
    if (n == 0) return PIMHIP_OK;
    rc = gemv_vm(st, (const half_t*)x, (const half_t*)A, nullptr, o, k, n, n, 0, static_cast<hipStream_t>(stream));
    if (rc != PIMHIP_OK) return rc;
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_execute_add(void* c, const void* a, const void* b, int64_t m, int64_t n, int b_broadcast, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!c || !a || !b) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "c, a and b must be non-null");
    if (m < 0 || n < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "m=%lld n=%lld must not be negative", (long long)m, (long long)n);
    const int64_t total = m * n;
    if (total == 0) return PIMHIP_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec_ok = (n % 8 == 0) && aligned16(a) && aligned16(b) && aligned16(c);
    if (vec_ok) {
        launch_add_f16_vec((const half_t*)a, (const half_t*)b, (half_t*)c, (long)(total / 8), (long)(n / 8), b_broadcast ? 1 : 0,
                           st->num_cus, s);
    } else {
        int64_t grid = (total + 255) / 256;
        if (grid > 8LL * st->num_cus) grid = 8LL * st->num_cus;
        add_f16_generic_kernel<<<(unsigned)grid, 256, 0, s>>>((const half_t*)a, (const half_t*)b, (half_t*)c, (long)total, (long)n,
                                                                b_broadcast ? 1 : 0);
    }
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}


extern "C" int pimhip_probe_stream_read(const void* data, int64_t bytes, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!data || bytes < 16 || bytes % 16 != 0 || !aligned16(data))
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "data must be 16-byte aligned and bytes a positive multiple of 16");
    const long n16 = (long)(bytes / 16);
    long grid = (n16 + 2047) / 2048;
    if (grid > 4L * st->num_cus) grid = 4L * st->num_cus;
    stream_read_probe_kernel<<<(unsigned)grid, 256, 0, static_cast<hipStream_t>(stream)>>>((const float4_probe_t*)data, n16, nullptr);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_execute_dot(void* out, const void* a, const void* b, int64_t in_w, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !a || !b) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, a and b must be non-null");
    if (in_w < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "in_w=%lld is negative", (long long)in_w);
    dot_f16_kernel<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>((const half_t*)a, (const half_t*)b, (half_t*)out, (long)in_w);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_execute_gemv_group(int count, void* const* outs, const void* const* ins,
                                         const void* const* weights, const void* const* biases,
                                         const int64_t* in_ws, const int64_t* out_ws, const int* acts, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (count < 0 || count > 64) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "count=%d not in [0, 64]", count);
    if (count == 0) return PIMHIP_OK;
    if (!outs || !ins || !weights || !in_ws || !out_ws) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "null array argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int done = 0;
    while (done < count) {
        GemvGroupArgs g;
        memset(&g, 0, sizeof(g));
        int n = 0, blocks = 0;
        unsigned long long weight_bytes = 0;
        for (; done + n < count && n < kGemvGroupMax; ++n) {
            const int i = done + n;
            if (!outs[i] || !ins[i] || !weights[i]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "entry %d has a null pointer", i);
            if (in_ws[i] < 0 || out_ws[i] < 1 || in_ws[i] > INT32_MAX || out_ws[i] > INT32_MAX)
                return fail(PIMHIP_ERR_INVALID_ARGUMENT, "entry %d: in_w=%lld out_w=%lld out of range", i, (long long)in_ws[i], (long long)out_ws[i]);
            if (in_ws[i] % 8 != 0 || !aligned16(weights[i]) || !aligned16(ins[i]))
                return fail(PIMHIP_ERR_UNSUPPORTED, "entry %d: grouped launch needs in_w %% 8 == 0 and 16-byte aligned in/weight", i);
            const int a = acts ? acts[i] : PIMHIP_ACT_NONE;
            if (a != PIMHIP_ACT_NONE && a != PIMHIP_ACT_RELU) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "entry %d: unknown activation %d", i, a);
            g.W[n] = (const half_t*)weights[i];
            g.x[n] = (const half_t*)ins[i];
            g.bias[n] = biases ? (const half_t*)biases[i] : nullptr;
            g.y[n] = (half_t*)outs[i];
            g.N[n] = (int)out_ws[i];
            g.K[n] = (int)in_ws[i];
            g.relu[n] = a == PIMHIP_ACT_RELU;
            g.block_begin[n] = blocks;
            weight_bytes += (unsigned long long)out_ws[i] * (unsigned long long)in_ws[i] * sizeof(half_t);
            const int rows_per_block = gemv_group_rows_per_block((int)in_ws[i]);
            blocks += ((int)out_ws[i] + rows_per_block - 1) / rows_per_block;
        }
        g.block_begin[n] = blocks;
        g.count = n;
        if (weight_bytes <= kKeepCachedBytes)
            gemv_mv_f16_group_kernel<true><<<blocks, kGemvGroupThreads, 0, s>>>(g);
        else
            gemv_mv_f16_group_kernel<false><<<blocks, kGemvGroupThreads, 0, s>>>(g);
        PIMHIP_HIP_CHECK(hipGetLastError());
        done += n;
    }
    return PIMHIP_OK;
}

