// The mixture-of-experts feed-forward step of the C ABI (include/pimhip.h): router, choice of the expert and its two
// products for one token in one launch.
#include "api_common.h"
#include "moe_kernels.h"

using namespace pimhip;

struct PimHipMoePlan {
    int device = 0;
    int num_experts = 0;
    int64_t d_model = 0, d_ff = 0;
    int act = 0;
    int scale_by_prob = 0;
    const half_t* router_w = nullptr;
    const half_t* router_b = nullptr;
    const half_t** tables = nullptr;       // device: [4][E] pointers (W1, b1, W2, b2 of every expert)
    unsigned long long* hx = nullptr;      // [2][kMoeMaxBlocks][kMoeEntryWords], all ones = empty
    unsigned int* g_counter = nullptr;     // [kMoeMaxBlocks][kMoeCounterStride]: every block's copy of the launch count
    unsigned int* abort_flag = nullptr;
    unsigned int* abort_host = nullptr;
    unsigned int* abort_host_dev = nullptr;
    unsigned int spin_limit = 1u << 22;
    bool reset_exchange = false;
    int blocks = 0;                        // workgroups of a step, all resident together
    int wpb = 1;                           // 16-byte words of hidden values per producing block
    int rpb2 = 1;                          // rows of W2 per block
    unsigned long long gave_up_events = 0; // waits that gave up, as far as the host has seen them (pimhip_moe_plan_fallbacks)
    bool alone = false;                    // every block computes all hidden values itself: after kMoeEventsBeforeAlone events
};

namespace
{
std::vector<PimHipMoePlan*> g_moe_plans;

constexpr size_t kMoeExchangeWords32 = (size_t)2 * kMoeMaxBlocks * kMoeEntryWords * 2;  // the exchange buffer as 32-bit words
constexpr unsigned long long kMoeEventsBeforeAlone = 3;  // waits given up before a plan stops exchanging for good

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

namespace pimhip
{
void destroy_all_moe_plans_locked()
{
    while (!g_moe_plans.empty()) destroy_moe_plan_locked(g_moe_plans.back());
}
}  // namespace pimhip

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
    // Hidden values travel as 16-byte words of eight, at most two per producing block; every block owns at most eight rows
    // of the second matrix.  The fewest blocks that allows: few, large participants shorten the all-to-all, which is what
    // bounds a step (768 / 3072: 192 blocks, two words and four rows each).
    const int nwords = (int)(d_ff / 8);
    int blocks = (nwords + kMoeMaxWordsPerBlock - 1) / kMoeMaxWordsPerBlock;
    const int blocks_for_w2 = (int)((d_model + kMoeMaxRows2 - 1) / kMoeMaxRows2);
    if (blocks < blocks_for_w2) blocks = blocks_for_w2;
    const int wpb_final = (nwords + blocks - 1) / blocks;
    int per_cu = 0;
    PIMHIP_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, moe_ffn_step_f16_kernel, kMoeThreads, 0));
    if ((int64_t)per_cu * st->num_cus < blocks)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the %d workgroups of the one-launch step cannot all be resident on this device", blocks);
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
    plan->blocks = blocks;
    plan->wpb = wpb_final;
    plan->rpb2 = (int)((d_model + blocks - 1) / blocks);
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
    launch_fill_u32(reinterpret_cast<unsigned int*>(plan->hx), kMoeExchangeWords32, ~0u, s);
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->g_counter), sizeof(unsigned int) * kMoeMaxBlocks * kMoeCounterStride));
    launch_fill_u32(plan->g_counter, (size_t)kMoeMaxBlocks * kMoeCounterStride, 0u, s);
    MOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->abort_flag), sizeof(unsigned int)));
    launch_fill_u32(plan->abort_flag, 1, 0u, s);
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
    // A wait that gave up no longer leaves anything undefined (the blocks complete the step by themselves): there is
    // nothing to report as an error.  pimhip_moe_plan_fallbacks counts the events.
    return PIMHIP_OK;
}

extern "C" int pimhip_moe_plan_fallbacks(PimHipMoePlan* plan, uint64_t* events, int* exchanging)
{
    if (!plan || !events) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and events must be non-null");
    *events = plan->gave_up_events + (*plan->abort_host != 0u ? 1u : 0u);
    if (exchanging) *exchanging = (plan->alone || *events >= kMoeEventsBeforeAlone) ? 0 : 1;
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
    if (*plan->abort_host != 0u && !capturing) {
        // A wait of an earlier step gave up.  That step's result was completed by the blocks themselves, and every step
        // since has run self-sufficient (the abort word stays up on the device); here, outside any capture, the exchange is
        // put back in order: drain the stream (steps sharing a plan are ordered on one stream), refill the slots, clear the
        // words.  A plan that has needed this kMoeEventsBeforeAlone times stops exchanging for good.
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        *plan->abort_host = 0u;
        ++plan->gave_up_events;
        if (plan->gave_up_events >= kMoeEventsBeforeAlone) plan->alone = true;
        launch_fill_u32(reinterpret_cast<unsigned int*>(plan->hx), kMoeExchangeWords32, ~0u, s);
        launch_fill_u32(plan->g_counter, (size_t)kMoeMaxBlocks * kMoeCounterStride, 0u, s);
        launch_fill_u32(plan->abort_flag, 1, 0u, s);
        PIMHIP_HIP_CHECK(hipGetLastError());
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
    a.wpb = plan->wpb;
    a.rpb2 = plan->rpb2;
    a.alone = plan->alone ? 1 : 0;
    // (every block publishes a word of hidden values unless the second matrix needs more blocks than there are words)
    a.count_stride = (int64_t)(plan->blocks - 1) * plan->wpb < plan->d_ff / 8 ? 0 : kMoeCounterStride;
    a.spin_limit = plan->spin_limit;
    // All blocks have to be resident at once, like the sequence kernel's: ordered after it on other streams.
    if (!capturing) {
        rc = order_after_previous_sequence_launch(st, s);
        if (rc != PIMHIP_OK) return rc;
    }
    moe_ffn_step_f16_kernel<<<dim3((unsigned)plan->blocks), dim3(kMoeThreads), 0, s>>>(a.x, a.router_w, a.router_b, a.tables, a.d_model, a.d_ff, a.E, a.act, a);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

