// Host-side state and helpers shared by the translation units behind the C ABI of include/pimhip.h.  Every kernel
// header of this directory is included by exactly one of them; what another unit needs of it is a launch function
// declared here.
#pragma once

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

#include "device_common.h"

namespace pimhip
{
// Records `fmt` as this thread's last error text and returns `status`.
int fail(int status, const char* fmt, ...);

#define PIMHIP_HIP_CHECK(expr)                                                                             \
    do {                                                                                                   \
        hipError_t e_ = (expr);                                                                            \
        if (e_ != hipSuccess) return fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- per-device state --------------------------------------------------------------------------
struct SplitWorkspace {
    float* partial = nullptr;            // [slices][N] fp32 records of the VM kernel; every word kVmEmpty between launches
    size_t partial_elems = 0;
    unsigned int* status = nullptr;      // pinned host word the kernel sets when a wait for a record gives up
    unsigned int* status_dev = nullptr;  // the same word as the device addresses it
    unsigned int* poison = nullptr;      // device word set at the same time: until it is cleared, reducing blocks ignore the records
    unsigned long long gave_up_events = 0;  // such events, as far as the host has seen them
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
    unsigned int* static_poison = nullptr;   // this device's copy of the poison word that goes with `scratch`
    unsigned long long static_gave_up_events = 0;
    // Polls of one record before a reducing lane of the sliced I_X_W kernel gives up (pimhip_set_gemv_spin_limit).
    unsigned int vm_spin_limit = 1u << 22;
};

extern std::mutex g_mutex;
int current_device_state(DeviceState** out);

// A launch whose workgroups wait for one another needs all of them resident at once.  Two such launches issued on
// different streams could each get part of the GPU and wait for the rest, so one on another stream than the device's
// previous one is ordered after it with an event (nothing is added while one stream is used).
int order_after_previous_sequence_launch(DeviceState* st, hipStream_t s);

// ---- small fills (api_core.hip) ------------------------------------------------------------------
// p[0 .. n) = v, as a kernel: a caller may be recording a graph, which must hold no memset node.
void launch_fill_u32(unsigned int* p, size_t n, unsigned int v, hipStream_t s);
// Up to six ranges of 32-bit words set to one value in one launch.
struct FillSegments {
    unsigned int* ptr[6];
    size_t words[6];
};
void launch_fill_segments(const FillSegments& seg, int count, unsigned int v, hipStream_t s);

// ---- api_gemv.hip -------------------------------------------------------------------------------
// c = a + b over total8 groups of eight fp16 values; b is one row of n8 groups added to every row when b_broadcast.
void launch_add_f16_vec(const half_t* a, const half_t* b, half_t* c, long total8, long n8, int b_broadcast, int num_cus, hipStream_t s);

// ---- api_xproj.hip ------------------------------------------------------------------------------
// out_p[T, N] = x[T, K] . w_p[N, K]^T + bias_p for p < count (1, or 2 for the two directions of a bidirectional layer).
int launch_input_projection(int count, float* const* out, const half_t* x, const half_t* const* w, const float* const* bias,
                            int64_t T, int64_t K, int64_t N, hipStream_t s, int64_t ldx = 0, int64_t ldw = 0);
// The same with weights in fragment order (launch_pack_w_fragments); N, K checked by the caller.  `ones`: n_ones ranges that
// the same launch sets to all-ones bytes with blocks of their own (a launch of their own where they are not whole
// 16-byte words).
int launch_input_projection_packed(int count, float* const* out, const half_t* x, const half_t* const* wp, const float* const* bias,
                                   int64_t T, int64_t K, int64_t N, int ksteps, hipStream_t s, const FillSegments* ones = nullptr,
                                   int n_ones = 0);
void packed_geometry(int64_t in_w, int64_t n_out, int* ntiles, int* ksteps);
void launch_pack_w_fragments(const half_t* w, half_t* packed, int64_t n_out, int64_t in_w, int ntiles, int ksteps, hipStream_t s);
// bsum[n] (fp32) = b_ih[n] + b_hh[n]; zeros for null biases.
void launch_lstm_bias_sum(const half_t* b_ih, const half_t* b_hh, float* bsum, int n, hipStream_t s);

// ---- plans: what pimhip_deinitialize destroys (each defined beside its plan type; g_mutex held) ---------------------
void destroy_all_lstm_plans_locked();
void destroy_all_decoder_plans_locked();
void destroy_all_moe_plans_locked();
void destroy_all_rnnt_plans_locked();

}  // namespace pimhip
