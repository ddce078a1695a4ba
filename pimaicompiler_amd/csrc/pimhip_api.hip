// C ABI of the gfx950 hot path (declared in include/pimhip.h): argument checking, kernel selection and
// launches.  No torch types, no library GEMM or RNN calls: every kernel launched here is in this directory.
#include "../../include/pimhip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "decoder_kernels.h"
#include "gemv_kernels.h"
#include "lstm_kernels.h"
#include "lstm_xcd_kernels.h"
#include "moe_kernels.h"
#include "shape_logic.h"
#include "xproj_kernels.h"

using namespace pimhip;

namespace
{
thread_local std::string g_last_error;

int fail(int status, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

#define PIMHIP_HIP_CHECK(expr)                                                                             \
    do {                                                                                                   \
        hipError_t e_ = (expr);                                                                            \
        if (e_ != hipSuccess) return fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Up to six ranges of 32-bit words set to one value in one launch (blockIdx.y = range).
struct FillSegments {
    unsigned int* ptr[6];
    size_t words[6];
};
__global__ void fill_segments_kernel(FillSegments seg, unsigned int v)
{
    unsigned int* p = seg.ptr[blockIdx.y];
    const size_t n = seg.words[blockIdx.y];
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

__global__ void fill_u32_kernel(unsigned int* p, size_t n, unsigned int v)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Partial-sum records of pimhip_execute_gemv_static, the entry point that allocates nothing: 256 KiB that every GPU
// the library runs on holds until the process ends.  In host code this name is only a stand-in for the symbol: the
// address a kernel can use is looked up once per device (pimhip_initialize) and kept in DeviceState::static_partial.
constexpr size_t kStaticScratchFloats = 64 * 1024;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

// ---- per-device state --------------------------------------------------------------------------
struct SplitWorkspace {
    float* partial = nullptr;            // [slices][N] fp32 records of the VM kernel; every word kVmEmpty between launches
    size_t partial_elems = 0;
    unsigned int* status = nullptr;      // pinned host word the kernel sets when a wait for a record gives up
    unsigned int* status_dev = nullptr;  // the same word as the device addresses it
};

struct DeviceState {
    bool initialized = false;
    int num_cus = 0;
    std::map<hipStream_t, SplitWorkspace> workspaces;  // one per stream: sibling GEMVs on different streams must not share
    // The persistent LSTM kernel needs all its blocks resident at once.  Two of them issued on different streams could
    // each get part of the GPU and wait for the rest forever, so a launch on another stream than the previous one is
    // ordered after it with an event (nothing is added while one stream is used).
    bool seq_launched = false;
    hipStream_t seq_stream = nullptr;
    hipEvent_t seq_event = nullptr;
    // pimhip_execute_gemv_static: this device's copy of `scratch` (every word kVmEmpty between launches) and the pinned
    // host word its kernel sets when a wait gives up, both set up by pimhip_initialize.
    float* static_partial = nullptr;
    unsigned int* static_status = nullptr;
    unsigned int* static_status_dev = nullptr;
    // Polls of one record before a reducing lane of the sliced I_X_W kernel gives up (pimhip_set_gemv_spin_limit).
    unsigned int vm_spin_limit = 1u << 22;
};

std::mutex g_mutex;
std::map<int, DeviceState> g_devices;

int current_device_state(DeviceState** out)
{
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_devices.find(dev);
    if (it == g_devices.end() || !it->second.initialized)
        return fail(PIMHIP_ERR_NOT_INITIALIZED, "device %d: pimhip_initialize has not been called", dev);
    *out = &it->second;
    return PIMHIP_OK;
}

int get_split_workspace(DeviceState* st, hipStream_t stream, size_t partial_elems, SplitWorkspace** out)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    SplitWorkspace& ws = st->workspaces[stream];
    const bool gave_up = ws.status && *ws.status != 0u;
    if (!ws.status || ws.partial_elems < partial_elems || gave_up) {
        // Allocation, synchronisation and the memset below are not for a graph: ask before touching anything.
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
        if (capture != hipStreamCaptureStatusNone)
            return fail(PIMHIP_ERR_UNSUPPORTED, "this I_X_W product needs its stream's workspace (re)allocated, which a graph must not "
                                                "record: run it once on this stream before the capture");
    }
    if (!ws.status) {
        PIMHIP_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&ws.status), sizeof(unsigned int), hipHostMallocMapped));
        *ws.status = 0u;
        PIMHIP_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&ws.status_dev), ws.status, 0));
    }
    if (ws.partial_elems < partial_elems || gave_up) {
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
        *ws.status = 0u;
        if (gave_up)
            return fail(PIMHIP_ERR_TIMEOUT, "an earlier GEMV on this stream gave up waiting for partial sums; its result is undefined "
                                            "(the workspace has been re-initialised, this call was not launched)");
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
int get_static_workspace(DeviceState* st, hipStream_t stream, size_t partial_elems, float** partial, unsigned int** status)
{
    if (!st->static_partial || !st->static_status)
        return fail(PIMHIP_ERR_NOT_INITIALIZED, "the static scratch buffer of this device has not been set up");
    if (partial_elems > kStaticScratchFloats)
        return fail(PIMHIP_ERR_UNSUPPORTED, "this I_X_W product needs %zu partial sums, the static scratch buffer holds %zu: "
                                            "use pimhip_execute_gemv", partial_elems, kStaticScratchFloats);
    if (*st->static_status != 0u) {
        // An earlier launch gave up a wait and may have left records behind: bring every word back to kVmEmpty with
        // a fill kernel on this stream (a caller may be recording a graph, which must hold no memset), launch nothing
        // else.  The word is cleared first: the launch that set it has ended, or the caller's calls overlap.
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
        if (capture != hipStreamCaptureStatusNone)
            return fail(PIMHIP_ERR_UNSUPPORTED, "an earlier static GEMV gave up a wait; its recovery is not for a graph");
        PIMHIP_HIP_CHECK(hipStreamSynchronize(stream));
        *st->static_status = 0u;
        fill_u32_kernel<<<(unsigned)(kStaticScratchFloats / 256), 256, 0, stream>>>(reinterpret_cast<unsigned int*>(st->static_partial),
                                                                                   kStaticScratchFloats, kVmEmpty);
        PIMHIP_HIP_CHECK(hipGetLastError());
        return fail(PIMHIP_ERR_TIMEOUT, "an earlier static GEMV gave up waiting for partial sums; its result is undefined "
                                        "(the scratch buffer has been re-initialised, this call was not launched)");
    }
    *partial = st->static_partial;
    *status = st->static_status_dev;
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
    if (slices > 1) {
        // Records of all slices but the last: partial[slice][N].
        const size_t partial_elems = (size_t)(slices - 1) * (size_t)N;
        int rc;
        if (static_ws) {
            rc = get_static_workspace(st, s, partial_elems, &partial, &status);
        } else {
            SplitWorkspace* ws = nullptr;
            rc = get_split_workspace(st, s, partial_elems, &ws);
            if (rc == PIMHIP_OK) {
                partial = ws->partial;
                status = ws->status_dev;
            }
        }
        if (rc != PIMHIP_OK) return rc;
    }
    dim3 grid(col_blocks, slices);
    gemv_vm_f16_kernel<WAVES, U, LPR><<<grid, WAVES * 64, 0, s>>>(x, A, bias, outs, (int)K, (int)N, (long)lda, relu,
                                                                    k_per_slice, partial, status, st->vm_spin_limit);
    return PIMHIP_OK;
}

}  // namespace

// ================================================================================================
// init / teardown
// ================================================================================================
struct PimHipLstmPlan;
struct PimHipDecoderPlan;
struct PimHipMoePlan;
namespace
{
std::vector<PimHipLstmPlan*> g_plans;
std::vector<PimHipDecoderPlan*> g_decoder_plans;
std::vector<PimHipMoePlan*> g_moe_plans;
int destroy_plan_locked(PimHipLstmPlan* plan);
int destroy_decoder_plan_locked(PimHipDecoderPlan* plan);
int destroy_moe_plan_locked(PimHipMoePlan* plan);
}  // namespace

extern "C" int pimhip_initialize(int device)
{
    int count = 0;
    PIMHIP_HIP_CHECK(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "device %d out of range [0, %d)", device, count);
    hipDeviceProp_t prop;
    PIMHIP_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(PIMHIP_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
    PIMHIP_HIP_CHECK(hipSetDevice(device));
    std::lock_guard<std::mutex> lock(g_mutex);
    DeviceState& st = g_devices[device];
    if (st.initialized) return PIMHIP_OK;
    st.num_cus = prop.multiProcessorCount;
    // The static scratch array of pimhip_execute_gemv_static: every GPU holds its own copy at its own address, so the
    // address is looked up with this device current, and the copy starts with every record empty.
    void* scratch_ptr = nullptr;
    PIMHIP_HIP_CHECK(hipGetSymbolAddress(&scratch_ptr, HIP_SYMBOL(scratch)));
    st.static_partial = static_cast<float*>(scratch_ptr);
    fill_u32_kernel<<<(unsigned)(kStaticScratchFloats / 256), 256, 0, nullptr>>>(reinterpret_cast<unsigned int*>(st.static_partial),
                                                                                kStaticScratchFloats, kVmEmpty);
    PIMHIP_HIP_CHECK(hipGetLastError());
    if (!st.static_status) {
        PIMHIP_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&st.static_status), sizeof(unsigned int), hipHostMallocMapped));
        PIMHIP_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&st.static_status_dev), st.static_status, 0));
    }
    *st.static_status = 0u;
    PIMHIP_HIP_CHECK(hipStreamSynchronize(nullptr));
    st.initialized = true;
    return PIMHIP_OK;
}

extern "C" const char* pimhip_last_error(void) { return g_last_error.c_str(); }

// ================================================================================================
// shape logic
// ================================================================================================
extern "C" int pimhip_gemm_broadcast(int64_t* shape1, int* rank1, int64_t* shape2, int* rank2)
{
    if (!shape1 || !shape2 || !rank1 || !rank2) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "null argument");
    if (*rank1 < 1 || *rank1 > 4 || *rank2 < 1 || *rank2 > 4)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ranks must be in [1, 4], got %d and %d", *rank1, *rank2);
    std::vector<int64_t> s1(shape1, shape1 + *rank1), s2(shape2, shape2 + *rank2);
    if (!gemm_broadcast(s1, s2)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "rank difference above 3");
    if (s1.size() > 4 || s2.size() > 4) return fail(PIMHIP_ERR_UNSUPPORTED, "broadcast produced a rank above 4");
    *rank1 = (int)s1.size();
    *rank2 = (int)s2.size();
    for (size_t i = 0; i < s1.size(); ++i) shape1[i] = s1[i];
    for (size_t i = 0; i < s2.size(); ++i) shape2[i] = s2[i];
    if (s1.size() != 4 || s2.size() != 4)
        return fail(PIMHIP_ERR_UNSUPPORTED, "shapes stay at ranks %zu and %zu, not 4", s1.size(), s2.size());
    return PIMHIP_OK;
}

extern "C" int pimhip_get_gemm_type(const int64_t* self_shape4, const int64_t* other_shape4, int* gemm_type)
{
    if (!self_shape4 || !other_shape4 || !gemm_type) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "null argument");
    *gemm_type = get_gemm_type(self_shape4, other_shape4);
    return PIMHIP_OK;
}

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
    // (the launch shapes of gemv_mv)
    if (out_w < 1024) {
        if (K >= 2048)
            gemv_mv_cat2_f16_kernel<1, 4, 4, 4><<<N, 256, 0, s>>>((const half_t*)weight, (const half_t*)in1, (const half_t*)in2, split,
                                                                    (const half_t*)bias, (half_t*)out, N, (int)K, (long)ldw, relu);
        else
            gemv_mv_cat2_f16_kernel<1, 2, 4, 4><<<N, 256, 0, s>>>((const half_t*)weight, (const half_t*)in1, (const half_t*)in2, split,
                                                                    (const half_t*)bias, (half_t*)out, N, (int)K, (long)ldw, relu);
    } else if (K >= 4096) {
        gemv_mv_cat2_f16_kernel<2, 4, 4, 4><<<(N + 1) / 2, 256, 0, s>>>((const half_t*)weight, (const half_t*)in1, (const half_t*)in2, split,
                                                                          (const half_t*)bias, (half_t*)out, N, (int)K, (long)ldw, relu);
    } else {
        gemv_mv_cat2_f16_kernel<2, 2, 4, 2><<<(N + 3) / 4, 256, 0, s>>>((const half_t*)weight, (const half_t*)in1, (const half_t*)in2, split,
                                                                          (const half_t*)bias, (half_t*)out, N, (int)K, (long)ldw, relu);
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
    // About 8 blocks per CU, each lane 16 bytes per operand and trip.
    const bool vec_ok = (n % 8 == 0) && aligned16(a) && aligned16(b) && aligned16(c);
    if (vec_ok) {
        const int64_t total8 = total / 8;
        int64_t grid = (total8 + 255) / 256;
        if (grid > 8LL * st->num_cus) grid = 8LL * st->num_cus;
        add_f16_vec_kernel<<<(unsigned)grid, 256, 0, s>>>((const half_t*)a, (const half_t*)b, (half_t*)c, (long)total8,
                                                            (long)(n / 8), b_broadcast ? 1 : 0);
    } else {
        int64_t grid = (total + 255) / 256;
        if (grid > 8LL * st->num_cus) grid = 8LL * st->num_cus;
        add_f16_generic_kernel<<<(unsigned)grid, 256, 0, s>>>((const half_t*)a, (const half_t*)b, (half_t*)c, (long)total, (long)n,
                                                                b_broadcast ? 1 : 0);
    }
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

namespace
{
__global__ void xcc_map_kernel(unsigned int* out)
{
    // HW_REG_XCC_ID (hardware register 20), bits 3:0
    if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;
}
}  // namespace

extern "C" int pimhip_probe_xcc_map(void* out, int blocks, int threads, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || blocks < 1 || threads < 1 || threads > 1024) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out must be non-null, blocks >= 1, threads in [1, 1024]");
    xcc_map_kernel<<<(unsigned)blocks, (unsigned)threads, 0, static_cast<hipStream_t>(stream)>>>(static_cast<unsigned int*>(out));
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
            const int rows_per_block = gemv_group_rows_per_block((int)in_ws[i]);
            blocks += ((int)out_ws[i] + rows_per_block - 1) / rows_per_block;
        }
        g.block_begin[n] = blocks;
        g.count = n;
        gemv_mv_f16_group_kernel<<<blocks, kGemvGroupThreads, 0, s>>>(g);
        PIMHIP_HIP_CHECK(hipGetLastError());
        done += n;
    }
    return PIMHIP_OK;
}

// ================================================================================================
// input projection
// ================================================================================================
namespace
{
// out_p[T, N] = x[T, K] . w_p[N, K]^T + bias_p for p < count (1, or 2 for the two directions of a bidirectional layer).
int launch_input_projection(int count, float* const* out, const half_t* x, const half_t* const* w, const float* const* bias,
                            int64_t T, int64_t K, int64_t N, hipStream_t s, int64_t ldx = 0, int64_t ldw = 0)
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

int launch_input_projection(float* out, const half_t* x, const half_t* w, const float* bias, int64_t T, int64_t K,
                            int64_t N, hipStream_t s)
{
    return launch_input_projection(1, &out, x, &w, &bias, T, K, N, s);
}

// The same with weights in fragment order (pack_w_fragments_kernel); N, K checked by the caller (plan creation).
int launch_input_projection_packed(int count, float* const* out, const half_t* x, const half_t* const* wp, const float* const* bias,
                                   int64_t T, int64_t K, int64_t N, int ksteps, hipStream_t s)
{
    if (T <= 0 || N <= 0) return PIMHIP_OK;
    XprojPackedProblems pr;
    memset(&pr, 0, sizeof(pr));
    for (int p = 0; p < count; ++p) {
        pr.wp[p] = wp[p];
        pr.bias[p] = bias[p];
        pr.out[p] = out[p];
    }
    const unsigned row_blocks = (unsigned)((T + kXprojTile - 1) / kXprojTile);
    auto blocks = [&](int cols) { return (unsigned)(((N + cols - 1) / cols + 7) / 8 * 8) * row_blocks; };
    // Measured on MI355X (T = 50, 200, 800; K = 240, 1024, 2048; N = 4096): with one row block 16-column tiles and
    // eight wavefronts splitting K; with more, 32-column tiles, and eight wavefronts only for long rows and few row blocks.
    if (row_blocks >= 2) {
        pr.blocks_per_problem = (int)blocks(32);
        if (row_blocks <= 4 && K >= 2048)
            input_projection_packed_f16_kernel<2, 8><<<blocks(32) * count, 512, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks);
        else
            input_projection_packed_f16_kernel<2, 4><<<blocks(32) * count, 256, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks);
    } else {
        pr.blocks_per_problem = (int)blocks(16);
        input_projection_packed_f16_kernel<1, 8><<<blocks(16) * count, 512, 0, s>>>(x, pr, (int)T, (int)K, (int)N, (long)K, ksteps, (int)row_blocks);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PIMHIP_ERR_HIP, "input projection launch failed: %s", hipGetErrorString(e));
    return PIMHIP_OK;
}
}  // namespace

extern "C" int pimhip_input_projection(void* out, const void* x, const void* w, const void* bias, int64_t seq_len,
                                       int64_t in_w, int64_t n_out, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!out || !x || !w) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "out, x and w must be non-null");
    if (seq_len < 0 || in_w < 0 || n_out < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "negative dimension");
    return launch_input_projection((float*)out, (const half_t*)x, (const half_t*)w, (const float*)bias, seq_len, in_w,
                                   n_out, static_cast<hipStream_t>(stream));
}

namespace
{
void packed_geometry(int64_t in_w, int64_t n_out, int* ntiles, int* ksteps)
{
    *ksteps = (int)((in_w + kXprojSlab - 1) / kXprojSlab * kXprojSlab / 32);
    *ntiles = (int)((n_out + 63) / 64 * 4);
}
}  // namespace

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
    const size_t chunks = (size_t)ntiles * ksteps * 64;
    pack_w_fragments_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
        (const half_t*)w, (half_t*)packed, (int)n_out, (int)in_w, (long)in_w, ntiles, ksteps);
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

// ================================================================================================
// LSTM
// ================================================================================================
struct PimHipLstmPlan {
    int device = -1;
    int num_cus = 0;
    int has_biases = 0;
    int num_layers = 0;
    int num_dirs = 1;
    int64_t input_size = 0;
    int64_t hidden = 0;
    int64_t max_seq_len = 0;
    int mode = 0;
    bool seq_kernel_ok = false;      // shape fits the persistent sequence kernel
    unsigned int spin_limit = 1u << 22;
    unsigned int* g_counters = nullptr;  // device, [kSeqMaxChains + 1]: per chain count, super-steps its region of hx has seen, plus 2
    size_t hx_region_words = 0;      // 32-bit words of one region of hx (one region per chain count)
    int max_wavefront = kSeqMaxChains;  // layers of a unidirectional stack advanced by one persistent launch
    int first_residual_layer = 1 << 30;  // layers from this one on give out_t = h_t + in_t (pimhip_lstm_plan_set_residual)
    bool xcd_res_ok = false;         // the pipeline kernel with residual sums is resident on this device

    struct Cell {
        const half_t* w_ih = nullptr;
        const half_t* w_hh = nullptr;
        const half_t* b_ih = nullptr;
        const half_t* b_hh = nullptr;
        float* bsum = nullptr;  // [4H] fp32, b_ih + b_hh (zeros when has_biases == 0)
        half_t* w_ih_packed = nullptr;  // w_ih in MFMA fragment order (cells whose projection runs as a batch), else null
        int ksteps = 0;                 // 32-wide K steps of the packed matrix
        int64_t in_w = 0;
    };
    std::vector<Cell> cells;          // index = layer * num_dirs + dir

    float* bsum_all = nullptr;        // backing store of every Cell::bsum
    std::vector<half_t*> packed;      // every Cell::w_ih_packed allocation
    float* xproj = nullptr;           // [num_dirs][max_seq_len][4H] fp32
    half_t* ybuf[2] = {nullptr, nullptr};  // inter-layer sequences [max_seq_len][num_dirs * H]
    float* c_state = nullptr;         // [num_dirs][H] fp32, per-step kernel's cell state
    unsigned int* hx = nullptr;       // [kSeqMaxChains][2][NB][kSeqEntryWords] exchange entries of the sequence kernel
    unsigned int* abort_flag = nullptr;
    unsigned int* abort_host = nullptr;      // pinned host word the kernel sets with the flag; read by pimhip_lstm_plan_status
    unsigned int* abort_host_dev = nullptr;  // the same word as the device addresses it
    int seq_blocks = 0;
    bool reset_exchange = false;     // the next forward starts from a cleared exchange buffer (layout change)
    bool seq_units8_ok = false;      // a single chain may run with 8 hidden units per block (half as many blocks)
    bool seq_wide = false;           // 1024 < H <= 2048: 32 columns per lane, eight units per block, one layer per launch
    // Mode 4: every recurrence on one XCD (lstm_xcd_f16_kernel).
    bool xcd_ok = false;             // H fits one XCD's registers and the device has the eight XCDs of 32 CUs the kernel assumes
    unsigned int* xcd_hx = nullptr;  // [kXcdMaxChains] regions of kXcdRegionWords, zero when the chain's counter is 2
    unsigned int* xcd_g_counters = nullptr;  // [kXcdMaxChains]
    unsigned int* xcd_claims = nullptr;      // [kXcdCount][kXcdMembers], zero when the counters are 2
    // Unidirectional stacks in mode 4 run as a pipeline over the XCDs: per boundary between two layers of a launch, the
    // lower layer's h per step ([max_seq_len][H] fp16) and the upper layer's projection rows ([max_seq_len][4H] fp32).
    unsigned char* xcd_pipe = nullptr;
    size_t xcd_pipe_boundary_bytes = 0;
};

namespace
{
int destroy_plan_locked(PimHipLstmPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    int prev = -1;
    hipGetDevice(&prev);
    hipSetDevice(plan->device);
    hipDeviceSynchronize();
    if (plan->bsum_all) hipFree(plan->bsum_all);
    for (half_t* q : plan->packed) hipFree(q);
    if (plan->xproj) hipFree(plan->xproj);
    if (plan->ybuf[0]) hipFree(plan->ybuf[0]);
    if (plan->ybuf[1]) hipFree(plan->ybuf[1]);
    if (plan->c_state) hipFree(plan->c_state);
    if (plan->hx) hipFree(plan->hx);
    if (plan->g_counters) hipFree(plan->g_counters);
    if (plan->xcd_hx) hipFree(plan->xcd_hx);
    if (plan->xcd_g_counters) hipFree(plan->xcd_g_counters);
    if (plan->xcd_claims) hipFree(plan->xcd_claims);
    if (plan->xcd_pipe) hipFree(plan->xcd_pipe);
    if (plan->abort_flag) hipFree(plan->abort_flag);
    if (plan->abort_host) hipHostFree(plan->abort_host);
    if (prev >= 0) hipSetDevice(prev);
    for (size_t i = 0; i < g_plans.size(); ++i) {
        if (g_plans[i] == plan) {
            g_plans.erase(g_plans.begin() + i);
            break;
        }
    }
    delete plan;
    return PIMHIP_OK;
}
}  // namespace

extern "C" int pimhip_deinitialize(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    while (!g_plans.empty()) destroy_plan_locked(g_plans.back());
    while (!g_decoder_plans.empty()) destroy_decoder_plan_locked(g_decoder_plans.back());
    while (!g_moe_plans.empty()) destroy_moe_plan_locked(g_moe_plans.back());
    int prev = -1;
    hipGetDevice(&prev);
    for (auto& kv : g_devices) {
        if (!kv.second.initialized) continue;
        hipSetDevice(kv.first);
        hipDeviceSynchronize();
        for (auto& w : kv.second.workspaces) {
            if (w.second.partial) hipFree(w.second.partial);
            if (w.second.status) hipHostFree(w.second.status);
        }
        kv.second.workspaces.clear();
        if (kv.second.static_status) hipHostFree(kv.second.static_status);
        if (kv.second.seq_event) hipEventDestroy(kv.second.seq_event);
        kv.second.initialized = false;
    }
    g_devices.clear();
    if (prev >= 0) hipSetDevice(prev);
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_create(PimHipLstmPlan** plan_out, const void* const* params, int n_params,
                                       int has_biases, int num_layers, int bidirectional, int64_t input_size,
                                       int64_t hidden_size, int64_t max_seq_len, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan_out || !params) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and params must be non-null");
    *plan_out = nullptr;
    if (num_layers < 1 || input_size < 1 || hidden_size < 1 || max_seq_len < 1)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "num_layers, input_size, hidden_size and max_seq_len must be positive");
    const int D = bidirectional ? 2 : 1;
    const int per_cell = has_biases ? 4 : 2;
    if (n_params != num_layers * D * per_cell)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "expected %d parameter tensors (layers=%d dirs=%d biases=%d), got %d",
                    num_layers * D * per_cell, num_layers, D, has_biases ? 1 : 0, n_params);
    for (int i = 0; i < n_params; ++i)
        if (!params[i]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "params[%d] is null", i);
    const int64_t H = hidden_size;
    if (H % 8 != 0 || input_size % 8 != 0)
        return fail(PIMHIP_ERR_UNSUPPORTED, "hidden_size (%lld) and input_size (%lld) must be multiples of 8", (long long)H, (long long)input_size);
    if (4 * H > INT32_MAX || input_size > INT32_MAX || max_seq_len > INT32_MAX || D * H > INT32_MAX)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "dimension above 2^31-1");

    hipStream_t s = static_cast<hipStream_t>(stream);
    int device = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&device));
    PimHipLstmPlan* plan = new PimHipLstmPlan();
    plan->device = device;
    plan->num_cus = st->num_cus;
    plan->has_biases = has_biases ? 1 : 0;
    plan->num_layers = num_layers;
    plan->num_dirs = D;
    plan->input_size = input_size;
    plan->hidden = H;
    plan->max_seq_len = max_seq_len;
    plan->cells.resize((size_t)num_layers * D);

    auto cleanup_fail = [&](int status) {
        std::lock_guard<std::mutex> lock(g_mutex);
        destroy_plan_locked(plan);
        return status;
    };
#define PLAN_HIP_CHECK(expr)                                                                                    \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) return cleanup_fail(fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_))); \
    } while (0)

    plan->seq_wide = H > kSeqMaxH && H <= kSeqMaxHWide;
    if (plan->seq_wide) plan->max_wavefront = 1;  // W_hh and W_ih of a second layer would not fit a wavefront's registers
    PLAN_HIP_CHECK(hipMalloc(&plan->bsum_all, sizeof(float) * 4 * H * plan->cells.size()));
    for (int l = 0; l < num_layers; ++l) {
        for (int d = 0; d < D; ++d) {
            const int ci = l * D + d;
            PimHipLstmPlan::Cell& c = plan->cells[ci];
            const void* const* p = params + (size_t)ci * per_cell;
            c.w_ih = (const half_t*)p[0];
            c.w_hh = (const half_t*)p[1];
            c.b_ih = has_biases ? (const half_t*)p[2] : nullptr;
            c.b_hh = has_biases ? (const half_t*)p[3] : nullptr;
            c.in_w = (l == 0) ? input_size : D * H;
            c.bsum = plan->bsum_all + (size_t)ci * 4 * H;
            if (!aligned16(c.w_ih) || !aligned16(c.w_hh))
                return cleanup_fail(fail(PIMHIP_ERR_UNSUPPORTED, "weights of layer %d direction %d are not 16-byte aligned", l, d));
            lstm_bias_sum_kernel<<<(unsigned)((4 * H + 255) / 256), 256, 0, s>>>(c.b_ih, c.b_hh, c.bsum, (int)(4 * H));
        }
    }
    PLAN_HIP_CHECK(hipGetLastError());
    // Cells whose input projection runs as a batch over the sequence (every layer of a bidirectional stack, the first
    // layer of every wavefront group of a unidirectional one) get a copy of w_ih in MFMA fragment order.
    for (int l = 0; l < num_layers; ++l) {
        if (D == 1 && l % plan->max_wavefront != 0) continue;
        for (int d = 0; d < D; ++d) {
            PimHipLstmPlan::Cell& c = plan->cells[(size_t)l * D + d];
            int ntiles = 0;
            packed_geometry(c.in_w, 4 * H, &ntiles, &c.ksteps);
            const size_t chunks = (size_t)ntiles * c.ksteps * 64;
            PLAN_HIP_CHECK(hipMalloc(&c.w_ih_packed, chunks * 16));
            plan->packed.push_back(c.w_ih_packed);
            pack_w_fragments_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, s>>>(c.w_ih, c.w_ih_packed, (int)(4 * H), (int)c.in_w,
                                                                                      (long)c.in_w, ntiles, c.ksteps);
        }
    }
    PLAN_HIP_CHECK(hipGetLastError());
    PLAN_HIP_CHECK(hipMalloc(&plan->xproj, sizeof(float) * (size_t)D * max_seq_len * 4 * H));
    if (num_layers > 1) {
        PLAN_HIP_CHECK(hipMalloc(&plan->ybuf[0], sizeof(half_t) * (size_t)max_seq_len * D * H));
        if (num_layers > 2) PLAN_HIP_CHECK(hipMalloc(&plan->ybuf[1], sizeof(half_t) * (size_t)max_seq_len * D * H));
    }
    PLAN_HIP_CHECK(hipMalloc(&plan->c_state, sizeof(float) * (size_t)D * H));
    PLAN_HIP_CHECK(hipMalloc(&plan->abort_flag, sizeof(unsigned int)));
    PLAN_HIP_CHECK(hipMemsetAsync(plan->abort_flag, 0, sizeof(unsigned int), s));
    // word 0: 1 = a wait gave up, 2 = a workgroup of the per-XCD kernel found its rank on its XCD taken (words 1 and 2
    // then hold that workgroup's index and the XCD it ran on)
    PLAN_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&plan->abort_host), 4 * sizeof(unsigned int), hipHostMallocMapped));
    plan->abort_host[0] = plan->abort_host[1] = plan->abort_host[2] = plan->abort_host[3] = 0;
    PLAN_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&plan->abort_host_dev), plan->abort_host, 0));

    // Persistent sequence kernel: one block per 4 hidden units (one unit per wavefront, weights in registers),
    // all blocks resident at once.
    plan->seq_blocks = (int)((H + kSeqUnits - 1) / kSeqUnits);
    plan->seq_kernel_ok = false;
    if (H <= kSeqMaxH) {
        int per_cu = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_seq_f16_kernel<kSeqMaxChains, true>, 256, 0));
        plan->seq_kernel_ok = (int64_t)per_cu * plan->num_cus >= plan->seq_blocks;
    } else if (plan->seq_wide) {
        int per_cu = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_seq_f16_kernel<2, false, 8, 32>, 512, 0));
        plan->seq_kernel_ok = (int64_t)per_cu * plan->num_cus >= (plan->seq_blocks + 1) / 2;
    }
    if (plan->seq_kernel_ok && !plan->seq_wide) {
        int per_cu8 = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu8, lstm_seq_f16_kernel<1, true, 8>, 512, 0));
        plan->seq_units8_ok = (int64_t)per_cu8 * plan->num_cus >= (plan->seq_blocks + 1) / 2;
    }
    if (plan->seq_kernel_ok) {
        // One region per number of chains a launch can advance: a launch writes exactly the words of its chains,
        // and the flag bits of a region must see every super-step that uses it.
        plan->hx_region_words = (size_t)2 * plan->seq_blocks * kSeqEntryWords;
        const size_t words = plan->hx_region_words * kSeqMaxChains;
        PLAN_HIP_CHECK(hipMalloc(&plan->hx, words * sizeof(unsigned int)));
        PLAN_HIP_CHECK(hipMemsetAsync(plan->hx, 0, words * sizeof(unsigned int), s));
        PLAN_HIP_CHECK(hipMalloc(&plan->g_counters, (kSeqMaxChains + 1) * sizeof(unsigned int)));
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counters, kSeqMaxChains + 1, 2u);
        PLAN_HIP_CHECK(hipGetLastError());
    }
    // One recurrence per XCD: the part this is written for has 8 XCDs of 32 CUs, a group is one workgroup per CU of one.
    if (H <= kXcdMaxH && plan->num_cus == kXcdCount * kXcdMembers) {
        int per_cu = 0;
        int per_cu_pipe = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_xcd_f16_kernel<false>, kXcdThreads, 0));
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_pipe, lstm_xcd_f16_kernel<true>, kXcdThreads, 0));
        plan->xcd_ok = per_cu >= 1 && per_cu_pipe >= 1;
        int per_cu_res = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_res, lstm_xcd_res_f16_kernel, kXcdThreads, 0));
        plan->xcd_res_ok = plan->xcd_ok && per_cu_res >= 1;
    }
    if (plan->xcd_ok) {
        const size_t words = (size_t)kXcdRegionWords * kXcdMaxChains;
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_hx, words * sizeof(unsigned int)));
        fill_u32_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(plan->xcd_hx, words, 0u);
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_g_counters, kXcdMaxChains * sizeof(unsigned int)));
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->xcd_g_counters, kXcdMaxChains, 2u);
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_claims, kXcdCount * kXcdMembers * sizeof(unsigned int)));
        fill_u32_kernel<<<1, 256, 0, s>>>(plan->xcd_claims, kXcdCount * kXcdMembers, 0u);
        PLAN_HIP_CHECK(hipGetLastError());
        if (D == 1 && num_layers >= 2) {
            plan->xcd_pipe_boundary_bytes = (size_t)max_seq_len * H * (sizeof(half_t) + 4 * sizeof(float));
            const int boundaries = (num_layers < kXcdMaxChains ? num_layers : kXcdMaxChains) - 1;
            PLAN_HIP_CHECK(hipMalloc(&plan->xcd_pipe, plan->xcd_pipe_boundary_bytes * boundaries));
        }
    }
    PLAN_HIP_CHECK(hipStreamSynchronize(s));
#undef PLAN_HIP_CHECK
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_plans.push_back(plan);
    }
    *plan_out = plan;
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_destroy(PimHipLstmPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    std::lock_guard<std::mutex> lock(g_mutex);
    bool known = false;
    for (PimHipLstmPlan* p : g_plans) known = known || (p == plan);
    if (!known) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown or already destroyed plan");
    return destroy_plan_locked(plan);
}

namespace
{
// Two workgroups of the one-recurrence-per-XCD kernel found themselves with the same rank on the same XCD: that launch's
// results are undefined, and the plan stops choosing that kernel by itself.
int xcd_placement_failure(PimHipLstmPlan* plan)
{
    plan->xcd_ok = false;
    if (plan->mode == 4) plan->mode = 0;
    return fail(PIMHIP_ERR_TIMEOUT, "the workgroups of the per-XCD LSTM kernel were not dealt to the XCDs in rotation (workgroup %u, on "
                                    "XCD %u, found its rank taken): the results of that forward are undefined; this plan uses the "
                                    "other kernels from now on",
                plan->abort_host[1], plan->abort_host[2]);
}
}  // namespace

extern "C" int pimhip_lstm_plan_set_mode(PimHipLstmPlan* plan, int mode)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    if (mode < 0 || mode > 4) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "mode %d not in {0, 1, 2, 3, 4}", mode);
    if ((mode == 2 || mode == 3) && !plan->seq_kernel_ok)
        return fail(PIMHIP_ERR_UNSUPPORTED, "hidden_size %lld does not fit the persistent sequence kernel", (long long)plan->hidden);
    if (mode == 4 && !plan->xcd_ok)
        return fail(PIMHIP_ERR_UNSUPPORTED, "hidden_size %lld does not fit one XCD's registers, or this device is not laid out as 8 XCDs of "
                                            "32 CUs", (long long)plan->hidden);
    // Modes 3 and 0 / 2 lay out a single chain's exchange entries differently: start over from a cleared buffer.
    if ((plan->mode == 3) != (mode == 3)) plan->reset_exchange = true;
    plan->mode = mode;
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_set_residual(PimHipLstmPlan* plan, int first_residual_layer)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    if (first_residual_layer < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "first_residual_layer=%d is negative", first_residual_layer);
    if (first_residual_layer < plan->num_layers) {
        if (plan->num_dirs != 1) return fail(PIMHIP_ERR_UNSUPPORTED, "residual sums are for unidirectional stacks");
        for (int l = first_residual_layer; l < plan->num_layers; ++l)
            if (plan->cells[(size_t)l].in_w != plan->hidden)
                return fail(PIMHIP_ERR_INVALID_ARGUMENT, "layer %d has input width %lld and hidden size %lld: its input cannot be added to its output",
                            l, (long long)plan->cells[(size_t)l].in_w, (long long)plan->hidden);
    }
    plan->first_residual_layer = first_residual_layer;
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_set_spin_limit(PimHipLstmPlan* plan, unsigned int spin_limit)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    plan->spin_limit = spin_limit;
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_status(PimHipLstmPlan* plan)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    if (*plan->abort_host != 0u) {
        // Reported once, here or by the next pimhip_lstm_forward, whichever comes first.  The caller has synchronised
        // the stream, so the kernel that set the word has ended and nothing sets it again after it is cleared.
        const bool misplaced = *plan->abort_host == 2u;
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        if (misplaced) return xcd_placement_failure(plan);
        return fail(PIMHIP_ERR_TIMEOUT, "a bounded wait of the persistent LSTM kernel gave up: the results of that forward are undefined");
    }
    return PIMHIP_OK;
}

namespace
{
int order_after_previous_sequence_launch(DeviceState* st, hipStream_t s)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    if (st->seq_launched && st->seq_stream != s) {
        if (!st->seq_event) PIMHIP_HIP_CHECK(hipEventCreateWithFlags(&st->seq_event, hipEventDisableTiming));
        // The event marks everything queued on the other stream so far, the earlier sequence kernel included.  That
        // stream may have been destroyed since: then there is nothing left to wait for.
        if (hipEventRecord(st->seq_event, st->seq_stream) == hipSuccess)
            PIMHIP_HIP_CHECK(hipStreamWaitEvent(s, st->seq_event, 0));
        else
            (void)hipGetLastError();
    }
    st->seq_launched = true;
    st->seq_stream = s;
    return PIMHIP_OK;
}
}  // namespace

extern "C" int pimhip_lstm_forward(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y,
                                   void* hn, void* cn, int64_t seq_len, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!h0 || !c0 || !hn || !cn) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "h0, c0, hn and cn must be non-null");
    if (seq_len > 0 && (!x || !y)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "x and y must be non-null when seq_len > 0");
    if (seq_len < 0 || seq_len > plan->max_seq_len)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "seq_len=%lld not in [0, max_seq_len=%lld]", (long long)seq_len, (long long)plan->max_seq_len);
    if (!aligned16(x) || !aligned16(h0) || !aligned16(y))
        return fail(PIMHIP_ERR_UNSUPPORTED, "x, h0 and y must be 16-byte aligned");

    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t H = plan->hidden;
    const int D = plan->num_dirs;
    const int L = plan->num_layers;
    const int64_t T = seq_len;
    const half_t* h0p = (const half_t*)h0;
    const half_t* c0p = (const half_t*)c0;
    half_t* hnp = (half_t*)hn;
    half_t* cnp = (half_t*)cn;

    if (T == 0) {
        // No step: the state passes through unchanged.
        PIMHIP_HIP_CHECK(hipMemcpyAsync(hn, h0, sizeof(half_t) * (size_t)L * D * H, hipMemcpyDeviceToDevice, s));
        PIMHIP_HIP_CHECK(hipMemcpyAsync(cn, c0, sizeof(half_t) * (size_t)L * D * H, hipMemcpyDeviceToDevice, s));
        return PIMHIP_OK;
    }

    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    // One step: the fused step kernel in every mode (the persistent kernel's hand-over of its step count to the next
    // launch needs two super-steps).
    // Automatic choice: one recurrence per XCD where its groups have something to run side by side or nothing to gain
    // from a wavefront (the two directions of a layer; a single unidirectional layer), the layer wavefront otherwise.
    // (Measured on MI355X, whole calls against the all-CU kernel: bidirectional layers 13-30 % faster from 16 steps on; a
    // single unidirectional layer 7-17 % from 16 steps at H <= 512 and from 64 at H = 1024; a unidirectional stack as a
    // pipeline over the XCDs 6-25 % for two layers from 32 steps, 12-60 % for three and more from 16.  Its 32 CUs per group
    // take longer to load the weights and the pipeline has to fill, which shorter sequences do not win back.)
    const bool xcd_pays = (D == 2 && T >= 16) || (D == 1 && L == 1 && T >= (H > 512 ? 64 : 16)) ||
                          (D == 1 && L >= 2 && T >= (L >= 3 ? 16 : 32));
    // (a stack with residual sums needs the pipeline kernel that makes them; where that one is not resident the stack runs
    // layer by layer on the other paths)
    const bool res_pipeline_missing = D == 1 && L >= 2 && plan->first_residual_layer < L && !plan->xcd_res_ok;
    const bool use_xcd = T >= 2 && T <= kSeqMaxT - 2 && plan->xcd_ok && !res_pipeline_missing &&
                         (plan->mode == 4 || (plan->mode == 0 && xcd_pays));
    const bool use_seq = !use_xcd && T >= 2 && T + kSeqMaxChains <= kSeqMaxT &&
                         (plan->mode == 2 || plan->mode == 3 || (plan->mode == 0 && plan->seq_kernel_ok));
    if (use_seq && !plan->seq_kernel_ok) return fail(PIMHIP_ERR_UNSUPPORTED, "persistent sequence kernel not available for this plan");
    if (*plan->abort_host != 0u) {
        // An earlier sequence kernel of this plan gave up a wait and nobody has asked pimhip_lstm_plan_status since:
        // the error is reported here instead of being dropped, and nothing is launched.  The word is cleared only
        // after the stream has drained (calls sharing a plan are ordered on one stream), so that kernel cannot set
        // it again; the next forward starts from a re-initialised exchange buffer.
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "an earlier forward of this plan gave up a wait; recovering from that is not for a "
                                                "graph: call pimhip_lstm_plan_status or one forward outside the capture first");
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        const bool misplaced = *plan->abort_host == 2u;
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        if (misplaced) return xcd_placement_failure(plan);
        return fail(PIMHIP_ERR_TIMEOUT, "an earlier forward of this plan gave up a wait of the persistent LSTM kernel: its results "
                                        "are undefined (this call was not launched; the next one starts from a re-initialised exchange buffer)");
    }
    if ((use_seq || use_xcd) && plan->reset_exchange) {
        // After a time-out or a change of the entry layout: re-arm the flag and bring the exchange buffer and its step
        // counters back to their initial state.
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "the plan's exchange buffer has to be re-initialised (after a time-out or a change of "
                                                "mode), which a graph must not record: run one forward outside the capture first");
        fill_u32_kernel<<<1, 1, 0, s>>>(plan->abort_flag, 1, 0u);
        if (plan->hx) {
            const size_t words = plan->hx_region_words * kSeqMaxChains;
            fill_u32_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(plan->hx, words, 0u);
            fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counters, kSeqMaxChains + 1, 2u);
        }
        if (plan->xcd_hx) {
            const size_t words = (size_t)kXcdRegionWords * kXcdMaxChains;
            fill_u32_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(plan->xcd_hx, words, 0u);
            fill_u32_kernel<<<1, 64, 0, s>>>(plan->xcd_g_counters, kXcdMaxChains, 2u);
            fill_u32_kernel<<<1, 256, 0, s>>>(plan->xcd_claims, kXcdCount * kXcdMembers, 0u);
        }
        PIMHIP_HIP_CHECK(hipGetLastError());
        plan->reset_exchange = false;
    }
    // seq_len == 1: fuse the input projection into the step (one launch per layer and direction).
    const bool fuse_xproj = !use_seq && T == 1;

    const half_t* layer_in = (const half_t*)x;
    const long y_stride = (long)D * H;
    auto residual = [&](int l) { return D == 1 && l >= plan->first_residual_layer; };
    // out = out + in over a whole sequence, for the paths that run a layer with a residual sum as a launch of its own
    auto add_input = [&](half_t* out, const half_t* in) {
        const long total8 = (long)T * H / 8;
        long grid = (total8 + 255) / 256;
        if (grid > 8L * st->num_cus) grid = 8L * st->num_cus;
        add_f16_vec_kernel<<<(unsigned)grid, 256, 0, s>>>(out, in, out, total8, (long)(H / 8), 0);
    };
    if (use_xcd) {
        // The groups of a launch have to be resident together, like the sequence kernel's blocks.
        if (!capturing) {
            rc = order_after_previous_sequence_launch(st, s);
            if (rc != PIMHIP_OK) return rc;
        }
        const int members = (int)((H + kXcdUnitsPerBlock - 1) / kXcdUnitsPerBlock);
        // A unidirectional stack: up to kXcdMaxChains layers per launch as a pipeline over the XCDs (recurrence of layer
        // j of the launch on XCD 2 j, the group that makes its projection rows from the layer below on XCD 2 j - 1).
        for (int l = 0; D == 1 && L >= 2 && l < L;) {
            const int n = (L - l) < kXcdMaxChains ? (L - l) : kXcdMaxChains;
            bool any_res = false;
            for (int j = 0; j < n; ++j) any_res = any_res || residual(l + j);
            if (any_res && !plan->xcd_res_ok) return fail(PIMHIP_ERR_UNSUPPORTED, "the pipeline kernel with residual sums is not resident on this device");
            const int last = l + n - 1;
            half_t* group_out = (last == L - 1) ? (half_t*)y : plan->ybuf[last & 1];
            const PimHipLstmPlan::Cell& cf = plan->cells[(size_t)l];
            if (cf.w_ih_packed) {
                float* outs1[1] = {plan->xproj};
                const half_t* ws1[1] = {cf.w_ih_packed};
                const float* bs1[1] = {cf.bsum};
                rc = launch_input_projection_packed(1, outs1, layer_in, ws1, bs1, T, cf.in_w, 4 * H, cf.ksteps, s);
            } else {
                rc = launch_input_projection(plan->xproj, layer_in, cf.w_ih, cf.bsum, T, cf.in_w, 4 * H, s);
            }
            if (rc != PIMHIP_OK) return rc;
            LstmXcdArgs a;
            memset(&a, 0, sizeof(a));
            FillSegments seg;
            memset(&seg, 0, sizeof(seg));
            for (int j = 0; j < n; ++j) {
                const int ci = l + j;
                XcdChain& ch = a.chain[j];
                ch.w_hh = plan->cells[ci].w_hh;
                ch.h0 = h0p + (size_t)ci * H;
                ch.c0 = c0p + (size_t)ci * H;
                ch.hn = hnp + (size_t)ci * H;
                ch.cn = cnp + (size_t)ci * H;
                ch.y = (j == n - 1) ? group_out : nullptr;
                a.role[2 * j] = j + 1;
                if (j == 0) {
                    ch.xproj = plan->xproj;
                    if (residual(ci)) ch.res_in = layer_in;
                } else {
                    unsigned char* boundary = plan->xcd_pipe + plan->xcd_pipe_boundary_bytes * (size_t)(j - 1);
                    half_t* seq = reinterpret_cast<half_t*>(boundary);
                    float* xp = reinterpret_cast<float*>(boundary + (size_t)plan->max_seq_len * H * sizeof(half_t));
                    a.chain[j - 1].seq_out = seq;
                    ch.xproj = xp;
                    ch.xproj_polled = 1;
                    if (residual(ci)) {
                        ch.res_in = seq;  // what the layer below hands up (its own residual sum included) is this layer's input
                        ch.res_polled = 1;
                    }
                    XcdProj& pj = a.proj[j - 1];
                    pj.w_ih = plan->cells[ci].w_ih;
                    pj.bsum = plan->cells[ci].bsum;
                    pj.seq_in = seq;
                    pj.xp_out = xp;
                    a.role[2 * j - 1] = kXcdRoleProj + (j - 1);
                    // this launch's slots start out as "not written yet": all-ones bytes
                    seg.ptr[2 * (j - 1)] = reinterpret_cast<unsigned int*>(seq);
                    seg.words[2 * (j - 1)] = (size_t)T * H / 2;
                    seg.ptr[2 * (j - 1) + 1] = reinterpret_cast<unsigned int*>(xp);
                    seg.words[2 * (j - 1) + 1] = (size_t)T * 4 * H;
                }
            }
            if (n > 1) fill_segments_kernel<<<dim3(64, 2 * (n - 1)), 256, 0, s>>>(seg, 0xffffffffu);
            a.hx = plan->xcd_hx;
            a.g_counter = plan->xcd_g_counters;
            a.claims = plan->xcd_claims;
            a.abort_flag = plan->abort_flag;
            a.abort_host = plan->abort_host_dev;
            a.y_stride = y_stride;
            a.H = (int)H;
            a.T = (int)T;
            a.spin_limit = plan->spin_limit;
            if (any_res)
                lstm_xcd_res_f16_kernel<<<dim3((unsigned)(kXcdCount * members)), dim3(kXcdThreads), 0, s>>>(a);
            else
                lstm_xcd_f16_kernel<true><<<dim3((unsigned)(kXcdCount * members)), dim3(kXcdThreads), 0, s>>>(a);
            PIMHIP_HIP_CHECK(hipGetLastError());
            layer_in = group_out;
            l += n;
        }
        for (int l = 0; (D == 2 || L == 1) && l < L; ++l) {
            half_t* layer_out = (l == L - 1) ? (half_t*)y : plan->ybuf[l & 1];
            const int64_t in_w = plan->cells[(size_t)l * D].in_w;
            const PimHipLstmPlan::Cell& c0 = plan->cells[(size_t)l * D];
            const PimHipLstmPlan::Cell& c1 = plan->cells[(size_t)l * D + (D - 1)];
            float* outs2[2] = {plan->xproj, plan->xproj + (size_t)plan->max_seq_len * 4 * H};
            const float* bs2[2] = {c0.bsum, c1.bsum};
            if (c0.w_ih_packed && c1.w_ih_packed) {
                const half_t* ws2[2] = {c0.w_ih_packed, c1.w_ih_packed};
                rc = launch_input_projection_packed(D, outs2, layer_in, ws2, bs2, T, in_w, 4 * H, c0.ksteps, s);
            } else {
                const half_t* ws2[2] = {c0.w_ih, c1.w_ih};
                rc = launch_input_projection(D, outs2, layer_in, ws2, bs2, T, in_w, 4 * H, s);
            }
            if (rc != PIMHIP_OK) return rc;
            LstmXcdArgs a;
            memset(&a, 0, sizeof(a));
            for (int d = 0; d < D; ++d) {
                const int ci = l * D + d;
                XcdChain& ch = a.chain[d];
                ch.w_hh = plan->cells[ci].w_hh;
                ch.xproj = outs2[d];
                ch.h0 = h0p + (size_t)ci * H;
                ch.c0 = c0p + (size_t)ci * H;
                ch.hn = hnp + (size_t)ci * H;
                ch.cn = cnp + (size_t)ci * H;
                ch.y = layer_out + (size_t)d * H;
                ch.reverse = d;
                a.role[d] = d + 1;  // direction d on XCD d
            }
            a.hx = plan->xcd_hx;
            a.g_counter = plan->xcd_g_counters;
            a.claims = plan->xcd_claims;
            a.abort_flag = plan->abort_flag;
            a.abort_host = plan->abort_host_dev;
            a.y_stride = y_stride;
            a.H = (int)H;
            a.T = (int)T;
            a.spin_limit = plan->spin_limit;
            lstm_xcd_f16_kernel<false><<<dim3((unsigned)(kXcdCount * members)), dim3(kXcdThreads), 0, s>>>(a);
            if (residual(l)) add_input(layer_out, layer_in);
            PIMHIP_HIP_CHECK(hipGetLastError());
            layer_in = layer_out;
        }
    } else if (use_seq) {
        // (Not on a capturing stream, where an event of another stream cannot be waited for: a caller who replays
        // graphs orders them against the device's other sequence launches.)
        if (!capturing) {
            rc = order_after_previous_sequence_launch(st, s);
            if (rc != PIMHIP_OK) return rc;
        }
        // Layers are taken in groups that one persistent launch advances together: the two directions of a
        // bidirectional layer, or up to kSeqMaxChains consecutive layers of a unidirectional stack as a wavefront.
        int l = 0;
        while (l < L) {
            int group_layers = (D == 2) ? 1 : ((L - l) < plan->max_wavefront ? (L - l) : plan->max_wavefront);
            if (D == 1) {
                // a layer with a residual sum runs alone: its input and its output both have to exist as sequences
                int gl = 1;
                while (!residual(l) && gl < group_layers && !residual(l + gl)) ++gl;
                group_layers = gl;
            }
            const int nc = (D == 2) ? 2 : group_layers;
            const int last = l + group_layers - 1;
            half_t* group_out = (last == L - 1) ? (half_t*)y : plan->ybuf[last & 1];
            const int64_t in_w = plan->cells[(size_t)l * D].in_w;
            LstmSeqArgs a;
            memset(&a, 0, sizeof(a));
            for (int k = 0; k < nc; ++k) {
                const int ci = (D == 2) ? (l * D + k) : (l + k);
                const PimHipLstmPlan::Cell& c = plan->cells[ci];
                LstmSeqChain& ch = a.chain[k];
                ch.w_hh = c.w_hh;
                ch.h0 = h0p + (size_t)ci * H;
                ch.c0 = c0p + (size_t)ci * H;
                ch.hn = hnp + (size_t)ci * H;
                ch.cn = cnp + (size_t)ci * H;
                if (D == 2 || k == 0) {
                    float* xp = plan->xproj + (size_t)((D == 2) ? k : 0) * plan->max_seq_len * 4 * H;
                    if (k == 0) {
                        // both directions of a bidirectional layer read the same x: one launch
                        const PimHipLstmPlan::Cell& c2 = plan->cells[(D == 2) ? ci + 1 : ci];
                        float* outs2[2] = {xp, xp + (size_t)plan->max_seq_len * 4 * H};
                        const float* bs2[2] = {c.bsum, c2.bsum};
                        if (c.w_ih_packed && c2.w_ih_packed) {
                            const half_t* ws2[2] = {c.w_ih_packed, c2.w_ih_packed};
                            rc = launch_input_projection_packed(D, outs2, layer_in, ws2, bs2, T, in_w, 4 * H, c.ksteps, s);
                        } else {
                            const half_t* ws2[2] = {c.w_ih, c2.w_ih};
                            rc = launch_input_projection(D, outs2, layer_in, ws2, bs2, T, in_w, 4 * H, s);
                        }
                        if (rc != PIMHIP_OK) return rc;
                    }
                    ch.xproj = xp;
                } else {
                    ch.w_ih = c.w_ih;
                    ch.bsum = c.bsum;
                }
                ch.reverse = (D == 2) ? k : 0;
                ch.y = (D == 2) ? group_out + (size_t)k * H : ((k == nc - 1) ? group_out : nullptr);
            }
            a.hx = plan->hx + plan->hx_region_words * (size_t)(nc - 1);
            a.abort_flag = plan->abort_flag;
            a.abort_host = plan->abort_host_dev;
            a.y_stride = y_stride;
            a.H = (int)H;
            a.T = (int)T;
            a.g_counter = plan->g_counters + nc;
            a.spin_limit = plan->spin_limit;
            const dim3 grid(plan->seq_blocks), block(256);
            if (plan->seq_wide) {
                const dim3 grid8((unsigned)((H + 7) / 8)), block8(512);
                if (D == 2)
                    lstm_seq_f16_kernel<2, false, 8, 32><<<grid8, block8, 0, s>>>(a);
                else
                    lstm_seq_f16_kernel<1, true, 8, 32><<<grid8, block8, 0, s>>>(a);  // max_wavefront == 1
            } else if (D == 2) {
                lstm_seq_f16_kernel<2, false><<<grid, block, 0, s>>>(a);
            } else {
                switch (nc) {
                    case 1:
                        // A single chain exchanges 2 bytes per unit: eight units per block still fit one 16-byte
                        // store and one 16-byte load per entry, and half as many blocks finish a round sooner.
                        if (plan->seq_units8_ok && plan->mode != 3)
                            lstm_seq_f16_kernel<1, true, 8><<<dim3((unsigned)((H + 7) / 8)), dim3(512), 0, s>>>(a);
                        else
                            lstm_seq_f16_kernel<1, true><<<grid, block, 0, s>>>(a);
                        break;
                    case 2: lstm_seq_f16_kernel<2, true><<<grid, block, 0, s>>>(a); break;
                    case 3: lstm_seq_f16_kernel<3, true><<<grid, block, 0, s>>>(a); break;
                    default: lstm_seq_f16_kernel<4, true><<<grid, block, 0, s>>>(a); break;
                }
            }
            if (residual(l)) add_input(group_out, layer_in);
            PIMHIP_HIP_CHECK(hipGetLastError());
            layer_in = group_out;
            l += group_layers;
        }
    } else {
        for (int l = 0; l < L; ++l) {
            half_t* layer_out = (l == L - 1) ? (half_t*)y : plan->ybuf[l & 1];
            const int64_t in_w = plan->cells[(size_t)l * D].in_w;
            for (int d = 0; d < D; ++d) {
                const int ci = l * D + d;
                const PimHipLstmPlan::Cell& c = plan->cells[ci];
                float* xp = plan->xproj + (size_t)d * plan->max_seq_len * 4 * H;
                half_t* yd = layer_out + (size_t)d * H;
                const half_t* h0c = h0p + (size_t)ci * H;
                const half_t* c0c = c0p + (size_t)ci * H;
                half_t* hnc = hnp + (size_t)ci * H;
                half_t* cnc = cnp + (size_t)ci * H;
                if (!fuse_xproj) {
                    rc = launch_input_projection(xp, layer_in, c.w_ih, c.bsum, T, in_w, 4 * H, s);
                    if (rc != PIMHIP_OK) return rc;
                }
                float* cst = plan->c_state + (size_t)d * H;
                const unsigned grid = (unsigned)((H + 3) / 4);
                for (int64_t step = 0; step < T; ++step) {
                    const int64_t t = d ? (T - 1 - step) : step;
                    const int64_t tp = d ? (t + 1) : (t - 1);
                    const half_t* h_prev = (step == 0) ? h0c : (yd + tp * y_stride);
                    const bool last = step == T - 1;
                    lstm_step_f16_kernel<4><<<grid, 256, 0, s>>>(
                        c.w_ih, c.w_hh, c.bsum, fuse_xproj ? nullptr : (xp + t * 4 * H), layer_in + t * in_w, h_prev,
                        (step == 0) ? c0c : nullptr, cst, yd + t * y_stride, last ? hnc : nullptr, last ? cnc : nullptr,
                        (int)in_w, (int)H);
                }
                PIMHIP_HIP_CHECK(hipGetLastError());
            }
            if (residual(l)) {
                add_input(layer_out, layer_in);
                PIMHIP_HIP_CHECK(hipGetLastError());
            }
            layer_in = layer_out;
        }
    }
    return PIMHIP_OK;
}

// ================================================================================================
// decoder step: a stack of seq_len-1 LSTM cells, the attention context, the residual sums and the classifier
// in one persistent launch
// ================================================================================================
struct PimHipDecoderPlan {
    int device = -1;
    int has_biases = 0;
    int num_layers = 0;
    int first_takes_context = 0;
    int first_residual_layer = 0;
    int64_t input_size = 0;
    int64_t hidden = 0;
    int64_t vocab = 0;
    const half_t* w_ih[kDecMaxLayers] = {};
    const half_t* w_hh[kDecMaxLayers] = {};
    const half_t* cls_w = nullptr;
    const half_t* cls_b = nullptr;
    float* bsum = nullptr;            // [num_layers][4H]
    float* cx_proj = nullptr;         // [num_layers][4H][enc_cap] fp32: W_ih[:, H:2H] . enc^T of the layers that take the context
    int64_t enc_cap = 0;              // encoder positions cx_proj has room for
    const half_t* enc = nullptr;      // the encoder outputs the projection was made from (read again only for ctx_outs)
    int64_t enc_len = 0;
    unsigned int* hx = nullptr;       // [kDecStages][blocks][kDecEntryWords], zero when *g_counter == 1
    unsigned int* g_counter = nullptr;
    unsigned int* abort_flag = nullptr;
    unsigned int* abort_host = nullptr;
    unsigned int* abort_host_dev = nullptr;
    unsigned int spin_limit = 1u << 22;
    int blocks = 0;
    bool reset_exchange = false;
};

namespace
{
int destroy_decoder_plan_locked(PimHipDecoderPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    int prev = -1;
    hipGetDevice(&prev);
    hipSetDevice(plan->device);
    hipDeviceSynchronize();
    if (plan->bsum) hipFree(plan->bsum);
    if (plan->cx_proj) hipFree(plan->cx_proj);
    if (plan->hx) hipFree(plan->hx);
    if (plan->g_counter) hipFree(plan->g_counter);
    if (plan->abort_flag) hipFree(plan->abort_flag);
    if (plan->abort_host) hipHostFree(plan->abort_host);
    if (prev >= 0) hipSetDevice(prev);
    for (size_t i = 0; i < g_decoder_plans.size(); ++i) {
        if (g_decoder_plans[i] == plan) {
            g_decoder_plans.erase(g_decoder_plans.begin() + i);
            break;
        }
    }
    delete plan;
    return PIMHIP_OK;
}

}  // namespace

extern "C" int pimhip_decoder_plan_create(PimHipDecoderPlan** plan_out, const void* const* params, int n_params, int has_biases,
                                          int num_layers, int first_takes_context, int first_residual_layer,
                                          int64_t input_size, int64_t hidden_size, const void* classifier_w,
                                          const void* classifier_b, int64_t vocab, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan_out || !params) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and params must be non-null");
    *plan_out = nullptr;
    if (num_layers < 1 || num_layers > kDecMaxLayers)
        return fail(PIMHIP_ERR_UNSUPPORTED, "a decoder step takes 1 to %d layers, got %d", kDecMaxLayers, num_layers);
    const int per_cell = has_biases ? 4 : 2;
    if (n_params != num_layers * per_cell)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "expected %d parameter tensors (layers=%d biases=%d), got %d", num_layers * per_cell,
                    num_layers, has_biases ? 1 : 0, n_params);
    for (int i = 0; i < n_params; ++i)
        if (!params[i]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "params[%d] is null", i);
    const int64_t H = hidden_size;
    if (H < 8 || H % 8 != 0 || H > kDecMaxH)
        return fail(PIMHIP_ERR_UNSUPPORTED, "hidden_size must be a multiple of 8 in [8, %d], got %lld", kDecMaxH, (long long)H);
    if (input_size < 8 || input_size % 8 != 0 || input_size > INT32_MAX / 8)
        return fail(PIMHIP_ERR_UNSUPPORTED, "input_size must be a positive multiple of 8, got %lld", (long long)input_size);
    if (first_takes_context && input_size != H)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "a first layer that takes cat(x, context) needs input_size == hidden_size");
    if (first_residual_layer < 0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "first_residual_layer is negative");
    if (first_residual_layer == 0 && input_size != H)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "a residual connection around layer 0 needs input_size == hidden_size");
    if (classifier_w && (vocab < 1 || vocab > INT32_MAX)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "vocab=%lld out of range", (long long)vocab);
    if (!classifier_w && classifier_b) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "classifier bias without classifier weight");
    for (int i = 0; i < num_layers; ++i)
        if (!aligned16(params[(size_t)i * per_cell]) || !aligned16(params[(size_t)i * per_cell + 1]))
            return fail(PIMHIP_ERR_UNSUPPORTED, "weights of layer %d are not 16-byte aligned", i);
    if (classifier_w && !aligned16(classifier_w)) return fail(PIMHIP_ERR_UNSUPPORTED, "the classifier weight is not 16-byte aligned");

    const int blocks = (int)((H + kDecUnits - 1) / kDecUnits);
    int per_cu = 0;
    PIMHIP_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decoder_step_f16_kernel<kDecMaxLayers, true>, kDecThreads, 0));
    if ((int64_t)per_cu * st->num_cus < blocks)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the %d blocks of the decoder step cannot all be resident on this device", blocks);

    hipStream_t s = static_cast<hipStream_t>(stream);
    int device = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&device));
    PimHipDecoderPlan* plan = new PimHipDecoderPlan();
    plan->device = device;
    plan->has_biases = has_biases ? 1 : 0;
    plan->num_layers = num_layers;
    plan->first_takes_context = first_takes_context ? 1 : 0;
    plan->first_residual_layer = first_residual_layer;
    plan->input_size = input_size;
    plan->hidden = H;
    plan->vocab = classifier_w ? vocab : 0;
    plan->cls_w = (const half_t*)classifier_w;
    plan->cls_b = (const half_t*)classifier_b;
    plan->blocks = blocks;
    auto cleanup_fail = [&](int status) {
        std::lock_guard<std::mutex> lock(g_mutex);
        destroy_decoder_plan_locked(plan);
        return status;
    };
#define DEC_HIP_CHECK(expr)                                                                                     \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) return cleanup_fail(fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_))); \
    } while (0)
    DEC_HIP_CHECK(hipMalloc(&plan->bsum, sizeof(float) * 4 * H * num_layers));
    for (int l = 0; l < num_layers; ++l) {
        const void* const* q = params + (size_t)l * per_cell;
        plan->w_ih[l] = (const half_t*)q[0];
        plan->w_hh[l] = (const half_t*)q[1];
        lstm_bias_sum_kernel<<<(unsigned)((4 * H + 255) / 256), 256, 0, s>>>(has_biases ? (const half_t*)q[2] : nullptr,
                                                                             has_biases ? (const half_t*)q[3] : nullptr,
                                                                             plan->bsum + (size_t)l * 4 * H, (int)(4 * H));
    }
    DEC_HIP_CHECK(hipGetLastError());
    const size_t words = (size_t)kDecStages * blocks * kDecEntryWords;
    DEC_HIP_CHECK(hipMalloc(&plan->hx, words * sizeof(unsigned int)));
    fill_u32_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(plan->hx, words, 0u);
    DEC_HIP_CHECK(hipMalloc(&plan->g_counter, sizeof(unsigned int)));
    fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counter, 1, 1u);
    DEC_HIP_CHECK(hipMalloc(&plan->abort_flag, sizeof(unsigned int)));
    fill_u32_kernel<<<1, 64, 0, s>>>(plan->abort_flag, 1, 0u);
    DEC_HIP_CHECK(hipGetLastError());
    DEC_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&plan->abort_host), sizeof(unsigned int), hipHostMallocMapped));
    *plan->abort_host = 0u;
    DEC_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&plan->abort_host_dev), plan->abort_host, 0));
    DEC_HIP_CHECK(hipStreamSynchronize(s));
#undef DEC_HIP_CHECK
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_decoder_plans.push_back(plan);
    }
    *plan_out = plan;
    return PIMHIP_OK;
}

#ifdef PIMHIP_DECODER_TRACE
namespace
{
unsigned long long* g_decoder_trace = nullptr;
}
extern "C" int pimhip_decoder_debug_set_trace(void* buffer)
{
    g_decoder_trace = static_cast<unsigned long long*>(buffer);
    return PIMHIP_OK;
}
#endif

extern "C" int pimhip_decoder_plan_destroy(PimHipDecoderPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    std::lock_guard<std::mutex> lock(g_mutex);
    bool known = false;
    for (PimHipDecoderPlan* q : g_decoder_plans) known = known || (q == plan);
    if (!known) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown or already destroyed decoder plan");
    return destroy_decoder_plan_locked(plan);
}

extern "C" int pimhip_decoder_plan_set_encoder(PimHipDecoderPlan* plan, const void* enc, int64_t enc_len, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!enc || enc_len < 1 || enc_len > INT32_MAX / 8) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "enc must be non-null and enc_len positive");
    if (!aligned16(enc)) return fail(PIMHIP_ERR_UNSUPPORTED, "enc must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t H = plan->hidden;
    const int L = plan->num_layers;
    if (enc_len > plan->enc_cap) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
        if (capture != hipStreamCaptureStatusNone)
            return fail(PIMHIP_ERR_UNSUPPORTED, "the plan's projection buffer has to grow for %lld encoder positions, which a graph must not "
                                                "record: call pimhip_decoder_plan_set_encoder once with that length before the capture", (long long)enc_len);
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));  // steps already queued may still read the old buffer
        if (plan->cx_proj) PIMHIP_HIP_CHECK(hipFree(plan->cx_proj));
        plan->cx_proj = nullptr;
        plan->enc_cap = 0;
        int64_t cap = enc_len < 64 ? 64 : enc_len;
        PIMHIP_HIP_CHECK(hipMalloc(&plan->cx_proj, sizeof(float) * (size_t)L * cap * 4 * H));
        plan->enc_cap = cap;
    }
    for (int l = 0; l < L; ++l) {
        if (!(l > 0 || plan->first_takes_context)) continue;
        // out[4H, S] = W_ih[:, H:2H] (4H rows of pitch 2H) . enc[S, H]^T: the kernel's "x" is the weight, its "w" the encoder
        // outputs, so that a gate row's S values are contiguous for the step kernel
        float* out = plan->cx_proj + (size_t)l * plan->enc_cap * 4 * H;
        const half_t* w = (const half_t*)enc;
        const float* no_bias = nullptr;
        rc = launch_input_projection(1, &out, plan->w_ih[l] + H, &w, &no_bias, 4 * H, H, enc_len, s, 2 * H, H);
        if (rc != PIMHIP_OK) return rc;
    }
    plan->enc = (const half_t*)enc;
    plan->enc_len = enc_len;
    return PIMHIP_OK;
}

extern "C" int pimhip_decoder_plan_set_spin_limit(PimHipDecoderPlan* plan, unsigned int spin_limit)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    plan->spin_limit = spin_limit;
    return PIMHIP_OK;
}

extern "C" int pimhip_decoder_plan_status(PimHipDecoderPlan* plan)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    if (*plan->abort_host != 0u) {
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        return fail(PIMHIP_ERR_TIMEOUT, "a bounded wait of the decoder step kernel gave up: the results of that step are undefined");
    }
    return PIMHIP_OK;
}

extern "C" int pimhip_decoder_step(PimHipDecoderPlan* plan, const void* x, const void* att, const void* ctx_in,
                                   const void* const* h_prev, const void* const* c_prev, void* const* hn,
                                   void* const* cn, void* const* layer_outs, void* const* ctx_outs, int n_ctx_outs, void* logits,
                                   void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!x || !h_prev || !c_prev || !hn || !cn) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "x, h_prev, c_prev, hn and cn must be non-null");
    const int L = plan->num_layers;
    const int64_t H = plan->hidden;
    bool any_ctx = false;
    for (int l = 0; l < L; ++l) any_ctx = any_ctx || l > 0 || plan->first_takes_context;
    // (every layer after the first takes cat(in, ctx) in this wiring)
    if (n_ctx_outs < 0 || n_ctx_outs > kDecMaxCtxOuts) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "n_ctx_outs=%d not in [0, %d]", n_ctx_outs, kDecMaxCtxOuts);
    if (n_ctx_outs > 0 && !ctx_outs) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ctx_outs is null");
    if ((any_ctx || n_ctx_outs > 0) && !ctx_in) {
        if (!att) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "the context needs ctx_in, or att");
        if (plan->enc_len < 1)
            return fail(PIMHIP_ERR_INVALID_ARGUMENT, "att needs the encoder outputs: call pimhip_decoder_plan_set_encoder first (once per sentence)");
    }
    if (plan->cls_w && !logits) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "logits must be non-null for a plan with a classifier");
    if (!aligned16(x)) return fail(PIMHIP_ERR_UNSUPPORTED, "x must be 16-byte aligned");
    if (ctx_in && (reinterpret_cast<uintptr_t>(ctx_in) & 3u)) return fail(PIMHIP_ERR_UNSUPPORTED, "ctx_in must be 4-byte aligned");

    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (*plan->abort_host != 0u) {
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "an earlier step of this plan gave up a wait; recovering from that is not for a graph");
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        return fail(PIMHIP_ERR_TIMEOUT, "an earlier step of this plan gave up a wait of the decoder step kernel: its results are undefined "
                                        "(this call was not launched; the next one starts from a re-initialised exchange buffer)");
    }
    if (plan->reset_exchange) {
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "the plan's exchange buffer has to be re-initialised after a time-out, which a graph must not "
                                                "record: run one step outside the capture first");
        const size_t words = (size_t)kDecStages * plan->blocks * kDecEntryWords;
        fill_u32_kernel<<<(unsigned)((words + 255) / 256), 256, 0, s>>>(plan->hx, words, 0u);
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counter, 1, 1u);
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->abort_flag, 1, 0u);
        PIMHIP_HIP_CHECK(hipGetLastError());
        plan->reset_exchange = false;
    }

    DecoderStepArgs a;
    memset(&a, 0, sizeof(a));
    a.n_layers = L;
    for (int l = 0; l < L; ++l) {
        if (!h_prev[l] || !c_prev[l] || !hn[l] || !cn[l]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "state pointers of layer %d are null", l);
        if (!aligned16(h_prev[l])) return fail(PIMHIP_ERR_UNSUPPORTED, "h_prev of layer %d must be 16-byte aligned", l);
        DecoderLayerArgs& ly = a.layer[l];
        ly.w_ih = plan->w_ih[l];
        ly.w_hh = plan->w_hh[l];
        ly.bsum = plan->bsum + (size_t)l * 4 * H;
        ly.h_prev = (const half_t*)h_prev[l];
        ly.c_prev = (const half_t*)c_prev[l];
        ly.hn = (half_t*)hn[l];
        ly.cn = (half_t*)cn[l];
        ly.out = layer_outs ? (half_t*)layer_outs[l] : nullptr;
        ly.takes_ctx = (l > 0 || plan->first_takes_context) ? 1 : 0;
        ly.cx_proj = (ly.takes_ctx && !ctx_in) ? plan->cx_proj + (size_t)l * plan->enc_cap * 4 * H : nullptr;
        ly.in_w = (int)(l == 0 ? (plan->first_takes_context ? 2 * H : plan->input_size) : 2 * H);
        ly.residual = l >= plan->first_residual_layer ? 1 : 0;
    }
    if (L == 1 && !plan->cls_w && (hn[0] == h_prev[0]))
        return fail(PIMHIP_ERR_UNSUPPORTED, "a one-layer step without a classifier cannot update its state in place");
    a.x = (const half_t*)x;
    a.x_w = (int)plan->input_size;
    a.ctx_in = (const half_t*)ctx_in;
    a.att = ctx_in ? nullptr : (const half_t*)att;
    a.enc = plan->enc;
    a.enc_len = ctx_in ? 0 : (int)plan->enc_len;
    a.n_ctx_out = n_ctx_outs;
    for (int o = 0; o < n_ctx_outs; ++o) {
        if (!ctx_outs[o] || (reinterpret_cast<uintptr_t>(ctx_outs[o]) & 3u)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ctx_outs[%d] is null or not 4-byte aligned", o);
        a.ctx_out[o] = (half_t*)ctx_outs[o];
    }
    a.cls_w = plan->cls_w;
    a.cls_b = plan->cls_b;
    a.logits = (half_t*)logits;
    a.vocab = (int)plan->vocab;
    a.hx = plan->hx;
    a.g_counter = plan->g_counter;
    a.abort_flag = plan->abort_flag;
    a.abort_host = plan->abort_host_dev;
    a.spin_limit = plan->spin_limit;
    a.H = (int)H;
#ifdef PIMHIP_DECODER_TRACE
    a.trace = g_decoder_trace;
#endif
    // All blocks have to be resident at once, like the sequence kernel's: ordered after it on other streams.
    if (!capturing) {
        rc = order_after_previous_sequence_launch(st, s);
        if (rc != PIMHIP_OK) return rc;
    }
    const dim3 grid(plan->blocks), block(kDecThreads);
    if (plan->cls_w) {
        switch (L) {
            case 1: decoder_step_f16_kernel<1, true><<<grid, block, 0, s>>>(a); break;
            case 2: decoder_step_f16_kernel<2, true><<<grid, block, 0, s>>>(a); break;
            case 3: decoder_step_f16_kernel<3, true><<<grid, block, 0, s>>>(a); break;
            default: decoder_step_f16_kernel<4, true><<<grid, block, 0, s>>>(a); break;
        }
    } else {
        switch (L) {
            case 1: decoder_step_f16_kernel<1, false><<<grid, block, 0, s>>>(a); break;
            case 2: decoder_step_f16_kernel<2, false><<<grid, block, 0, s>>>(a); break;
            case 3: decoder_step_f16_kernel<3, false><<<grid, block, 0, s>>>(a); break;
            default: decoder_step_f16_kernel<4, false><<<grid, block, 0, s>>>(a); break;
        }
    }
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

// ================================================================================================
// a token's pass through a top-1 mixture-of-experts feed-forward block, one launch (moe_kernels.h)
// ================================================================================================
struct PimHipMoePlan {
    int device = 0;
    int num_experts = 0;
    int64_t d_model = 0, d_ff = 0;
    int act = 0;
    int scale_by_prob = 0;
    const half_t* router_w = nullptr;
    const half_t* router_b = nullptr;
    const half_t** tables = nullptr;       // device: [4][E] pointers (W1, b1, W2, b2 of every expert)
    unsigned long long* hx = nullptr;      // [2][kMoeBlocks][kMoeEntryWords], all ones = empty
    unsigned int* g_counter = nullptr;
    unsigned int* abort_flag = nullptr;
    unsigned int* abort_host = nullptr;
    unsigned int* abort_host_dev = nullptr;
    unsigned int spin_limit = 1u << 22;
    bool reset_exchange = false;
};

namespace
{
constexpr size_t kMoeExchangeWords32 = (size_t)2 * kMoeBlocks * kMoeEntryWords * 2;  // the exchange buffer as 32-bit words

int destroy_moe_plan_locked(PimHipMoePlan* plan)
{
    if (!plan) return PIMHIP_OK;
    int prev = -1;
    hipGetDevice(&prev);
    hipSetDevice(plan->device);
    hipDeviceSynchronize();
    if (plan->tables) hipFree(plan->tables);
    if (plan->hx) hipFree(plan->hx);
    if (plan->g_counter) hipFree(plan->g_counter);
    if (plan->abort_flag) hipFree(plan->abort_flag);
    if (plan->abort_host) hipHostFree(plan->abort_host);
    if (prev >= 0) hipSetDevice(prev);
    for (size_t i = 0; i < g_moe_plans.size(); ++i) {
        if (g_moe_plans[i] == plan) {
            g_moe_plans.erase(g_moe_plans.begin() + i);
            break;
        }
    }
    delete plan;
    return PIMHIP_OK;
}
}  // namespace

extern "C" int pimhip_moe_plan_create(PimHipMoePlan** plan_out, const void* router_w, const void* router_b,
                                      const void* const* w1, const void* const* b1, const void* const* w2,
                                      const void* const* b2, int num_experts, int64_t d_model, int64_t d_ff, int act,
                                      int scale_by_router_prob, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan_out || !router_w || !w1 || !w2) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan, router_w, w1 and w2 must be non-null");
    if (num_experts < 1 || num_experts > kMoeMaxExperts)
        return fail(PIMHIP_ERR_UNSUPPORTED, "num_experts=%d not in [1, %d]", num_experts, kMoeMaxExperts);
    if (d_model < 8 || d_model > kMoeMaxModel || (d_model & 7) || d_ff < 8 || d_ff > kMoeMaxFf || (d_ff & 7))
        return fail(PIMHIP_ERR_UNSUPPORTED, "the one-launch step takes d_model in [8, %d] and d_ff in [8, %d], multiples of 8 (got %lld, %lld): "
                                            "use three pimhip_execute_gemv calls", kMoeMaxModel, kMoeMaxFf, (long long)d_model, (long long)d_ff);
    if (act != PIMHIP_ACT_NONE && act != PIMHIP_ACT_RELU) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "act=%d", act);
    if (st->num_cus < kMoeBlocks)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the one-launch step needs %d compute units resident at once (device has %d)", kMoeBlocks, st->num_cus);
    if (!aligned16(router_w)) return fail(PIMHIP_ERR_UNSUPPORTED, "router_w must be 16-byte aligned");
    std::vector<const half_t*> host_tables((size_t)4 * num_experts, nullptr);
    for (int e = 0; e < num_experts; ++e) {
        if (!w1[e] || !w2[e]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "w1[%d] / w2[%d] is null", e, e);
        if (!aligned16(w1[e]) || !aligned16(w2[e])) return fail(PIMHIP_ERR_UNSUPPORTED, "the weights of expert %d must be 16-byte aligned", e);
        host_tables[(size_t)0 * num_experts + e] = (const half_t*)w1[e];
        host_tables[(size_t)1 * num_experts + e] = b1 ? (const half_t*)b1[e] : nullptr;
        host_tables[(size_t)2 * num_experts + e] = (const half_t*)w2[e];
        host_tables[(size_t)3 * num_experts + e] = b2 ? (const half_t*)b2[e] : nullptr;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    PimHipMoePlan* plan = new PimHipMoePlan();
    PIMHIP_HIP_CHECK(hipGetDevice(&plan->device));
    plan->num_experts = num_experts;
    plan->d_model = d_model;
    plan->d_ff = d_ff;
    plan->act = act;
    plan->scale_by_prob = scale_by_router_prob ? 1 : 0;
    plan->router_w = (const half_t*)router_w;
    plan->router_b = (const half_t*)router_b;
    auto cleanup_fail = [&](int status) {
        std::lock_guard<std::mutex> lock(g_mutex);
        destroy_moe_plan_locked(plan);
        return status;
    };
#define MOE_HIP_CHECK(expr)                                                                                     \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) return cleanup_fail(fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_))); \
    } while (0)
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->tables), host_tables.size() * sizeof(const half_t*)));
    MOE_HIP_CHECK(hipMemcpyAsync(plan->tables, host_tables.data(), host_tables.size() * sizeof(const half_t*), hipMemcpyHostToDevice, s));
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->hx), kMoeExchangeWords32 * sizeof(unsigned int)));
    fill_u32_kernel<<<(unsigned)((kMoeExchangeWords32 + 255) / 256), 256, 0, s>>>(reinterpret_cast<unsigned int*>(plan->hx), kMoeExchangeWords32, ~0u);
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->g_counter), sizeof(unsigned int)));
    fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counter, 1, 0u);
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->abort_flag), sizeof(unsigned int)));
    fill_u32_kernel<<<1, 64, 0, s>>>(plan->abort_flag, 1, 0u);
    MOE_HIP_CHECK(hipGetLastError());
    MOE_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&plan->abort_host), sizeof(unsigned int), hipHostMallocMapped));
    *plan->abort_host = 0u;
    MOE_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&plan->abort_host_dev), plan->abort_host, 0));
    MOE_HIP_CHECK(hipStreamSynchronize(s));  // (host_tables goes out of scope)
#undef MOE_HIP_CHECK
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_moe_plans.push_back(plan);
    }
    *plan_out = plan;
    return PIMHIP_OK;
}

extern "C" int pimhip_moe_plan_destroy(PimHipMoePlan* plan)
{
    if (!plan) return PIMHIP_OK;
    std::lock_guard<std::mutex> lock(g_mutex);
    bool known = false;
    for (PimHipMoePlan* q : g_moe_plans) known = known || (q == plan);
    if (!known) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown or already destroyed mixture-of-experts plan");
    return destroy_moe_plan_locked(plan);
}

extern "C" int pimhip_moe_plan_set_spin_limit(PimHipMoePlan* plan, unsigned int spin_limit)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    plan->spin_limit = spin_limit;
    return PIMHIP_OK;
}

extern "C" int pimhip_moe_plan_status(PimHipMoePlan* plan)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    if (*plan->abort_host != 0u) {
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        return fail(PIMHIP_ERR_TIMEOUT, "a bounded wait of the mixture-of-experts step kernel gave up: the results of that step are undefined");
    }
    return PIMHIP_OK;
}

extern "C" int pimhip_moe_ffn_step(PimHipMoePlan* plan, const void* x, void* y, void* router_logits, int* expert, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!x || !y) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "x and y must be non-null");
    if (!aligned16(x)) return fail(PIMHIP_ERR_UNSUPPORTED, "x must be 16-byte aligned");
    if (expert && (reinterpret_cast<uintptr_t>(expert) & 3u)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "expert must be 4-byte aligned");

    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (*plan->abort_host != 0u) {
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "an earlier step of this plan gave up a wait; recovering from that is not for a graph");
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        return fail(PIMHIP_ERR_TIMEOUT, "an earlier step of this plan gave up a wait of the mixture-of-experts step kernel: its results are "
                                        "undefined (this call was not launched; the next one starts from a re-initialised exchange buffer)");
    }
    if (plan->reset_exchange) {
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "the plan's exchange buffer has to be re-initialised after a time-out, which a graph must not "
                                                "record: run one step outside the capture first");
        fill_u32_kernel<<<(unsigned)((kMoeExchangeWords32 + 255) / 256), 256, 0, s>>>(reinterpret_cast<unsigned int*>(plan->hx), kMoeExchangeWords32, ~0u);
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->g_counter, 1, 0u);
        fill_u32_kernel<<<1, 64, 0, s>>>(plan->abort_flag, 1, 0u);
        PIMHIP_HIP_CHECK(hipGetLastError());
        plan->reset_exchange = false;
    }
    MoeStepArgs a;
    memset(&a, 0, sizeof(a));
    a.x = (const half_t*)x;
    a.router_w = plan->router_w;
    a.router_b = plan->router_b;
    a.tables = plan->tables;
    a.y = (half_t*)y;
    a.router_logits = (half_t*)router_logits;
    a.expert = expert;
    a.hx = plan->hx;
    a.g_counter = plan->g_counter;
    a.abort_flag = plan->abort_flag;
    a.abort_host = plan->abort_host_dev;
    a.d_model = (int)plan->d_model;
    a.d_ff = (int)plan->d_ff;
    a.E = plan->num_experts;
    a.act = plan->act;
    a.scale_by_prob = plan->scale_by_prob;
    a.rpb1 = (int)((plan->d_ff + kMoeBlocks - 1) / kMoeBlocks);
    a.rpb2 = (int)((plan->d_model + kMoeBlocks - 1) / kMoeBlocks);
    a.spin_limit = plan->spin_limit;
    // All blocks have to be resident at once, like the sequence kernel's: ordered after it on other streams.
    if (!capturing) {
        rc = order_after_previous_sequence_launch(st, s);
        if (rc != PIMHIP_OK) return rc;
    }
    moe_ffn_step_f16_kernel<<<dim3(kMoeBlocks), dim3(kMoeThreads), 0, s>>>(a);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}
