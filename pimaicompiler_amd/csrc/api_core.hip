// Initialisation and teardown, the error text, the shape logic and the small fills: the part of the C ABI of
// include/pimhip.h that belongs to no kernel family.
#include "api_common.h"
#include "shape_logic.h"

namespace pimhip
{
namespace
{
thread_local std::string g_last_error;

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
// Non-zero from the moment a reducing block of pimhip_execute_gemv_static has given up on a record until the host has
// refilled `scratch`: while it is up, reducing blocks ignore the records (one that arrived late would pass for the next
// launch's) and compute every slice themselves.
static __device__ unsigned int scratch_poison;

std::map<int, DeviceState> g_devices;
}  // namespace

std::mutex g_mutex;

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

void launch_fill_u32(unsigned int* p, size_t n, unsigned int v, hipStream_t s)
{
    if (n == 0) return;
    fill_u32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p, n, v);
}

void launch_fill_segments(const FillSegments& seg, int count, unsigned int v, hipStream_t s)
{
    if (count < 1) return;
    fill_segments_kernel<<<dim3(64, (unsigned)count), 256, 0, s>>>(seg, v);
}

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
}  // namespace pimhip

using namespace pimhip;

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
    launch_fill_u32(reinterpret_cast<unsigned int*>(st.static_partial), kStaticScratchFloats, kVmEmpty, nullptr);
    void* poison_ptr = nullptr;
    PIMHIP_HIP_CHECK(hipGetSymbolAddress(&poison_ptr, HIP_SYMBOL(scratch_poison)));
    st.static_poison = static_cast<unsigned int*>(poison_ptr);
    launch_fill_u32(st.static_poison, 1, 0u, nullptr);
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

extern "C" int pimhip_deinitialize(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    destroy_all_lstm_plans_locked();
    destroy_all_decoder_plans_locked();
    destroy_all_moe_plans_locked();
    destroy_all_rnnt_plans_locked();
    int prev = -1;
    hipGetDevice(&prev);
    for (auto& kv : g_devices) {
        if (!kv.second.initialized) continue;
        hipSetDevice(kv.first);
        hipDeviceSynchronize();
        for (auto& w : kv.second.workspaces) {
            if (w.second.partial) hipFree(w.second.partial);
            if (w.second.poison) hipFree(w.second.poison);
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

// ================================================================================================
// shape logic
// ================================================================================================
extern "C" int pimhip_gemm_broadcast(int64_t* shape1, int* rank1, int64_t* shape2, int* rank2)
{
    if (!shape1 || !shape2 || !rank1 || !rank2) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "null argument");
    if (*rank1 < 1 || *rank1 > 4 || *rank2 < 1 || *rank2 > 4)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "ranks must be in [1, 4], got %d and %d", *rank1, *rank2);
    SmallShape s1, s2;
    s1.n = *rank1;
    s2.n = *rank2;
    for (int i = 0; i < s1.n; ++i) s1[i] = shape1[i];
    for (int i = 0; i < s2.n; ++i) s2[i] = shape2[i];
    if (!gemm_broadcast(s1, s2)) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "rank difference above 3");
    if (s1.n > 4 || s2.n > 4) return fail(PIMHIP_ERR_UNSUPPORTED, "broadcast produced a rank above 4");
    *rank1 = s1.n;
    *rank2 = s2.n;
    for (int i = 0; i < s1.n; ++i) shape1[i] = s1[i];
    for (int i = 0; i < s2.n; ++i) shape2[i] = s2[i];
    if (s1.n != 4 || s2.n != 4)
        return fail(PIMHIP_ERR_UNSUPPORTED, "shapes stay at ranks %d and %d, not 4", s1.n, s2.n);
    return PIMHIP_OK;
}

extern "C" int pimhip_get_gemm_type(const int64_t* self_shape4, const int64_t* other_shape4, int* gemm_type)
{
    if (!self_shape4 || !other_shape4 || !gemm_type) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "null argument");
    *gemm_type = get_gemm_type(self_shape4, other_shape4);
    return PIMHIP_OK;
}
