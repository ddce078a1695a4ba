// The RNN-transducer entry points of the C ABI (include/pimhip.h): one step of the greedy decoding loop (the prediction
// network's LSTM cells at seq_len 1 and the joint network's two products) in one launch, and the whole loop over an
// utterance in one launch.
#include "api_common.h"
#include "rnnt_greedy_kernels.h"

using namespace pimhip;

struct PimHipRnntPlan {
    int device = -1;
    int num_layers = 0;
    int64_t input_size = 0, hidden = 0, enc_size = 0, joint_size = 0, vocab = 0;
    const half_t* w_ih[kRnntMaxLayers] = {};
    const half_t* w_hh[kRnntMaxLayers] = {};
    const half_t* w1 = nullptr;
    const half_t* b1 = nullptr;
    const half_t* w2 = nullptr;
    const half_t* b2 = nullptr;
    float* bsum = nullptr;                 // [num_layers][4H], or null without biases
    unsigned long long* hx = nullptr;      // [2][blocks][kRnntEntryWords], all ones = empty
    unsigned int* g_counter = nullptr;     // [blocks][kRnntCounterStride]
    unsigned int* greedy = nullptr;        // what the loop kernel exchanges through, refilled before every launch of it:
                                           // [kRnntGreedySets][blocks][kRnntEntryWords] 8-byte words (all ones), then
                                           // seen [blocks][kRnntSeenStride] and solo_owner (zero)
    bool greedy_resident = false;          // all workgroups of the loop kernel fit on the device together
    unsigned int* abort_flag = nullptr;
    unsigned int* abort_host = nullptr;
    unsigned int* abort_host_dev = nullptr;
    unsigned int spin_limit = 1u << 22;
    int blocks = 0;                        // workgroups of a step, all resident together
    unsigned long long gave_up_events = 0; // waits that gave up, as far as the host has seen them (pimhip_rnnt_plan_fallbacks)
    bool alone = false;                    // every block computes what it needs by itself: after kRnntEventsBeforeAlone events
};

namespace
{
std::vector<PimHipRnntPlan*> g_rnnt_plans;

constexpr unsigned long long kRnntEventsBeforeAlone = 3;  // waits given up before a plan stops exchanging for good

size_t exchange_words32(const PimHipRnntPlan* plan) { return (size_t)2 * plan->blocks * kRnntEntryWords * 2; }
size_t greedy_exchange_words32(const PimHipRnntPlan* plan)
{
    const size_t n_lstm = (size_t)plan->num_layers * (plan->hidden / 8), n_joint = plan->joint_size / 8, n_vocab = (plan->vocab + 7) / 8;
    return (kRnntGreedyVersions * n_lstm + kRnntGreedyRing * (n_joint + n_vocab)) * kRnntEntryWords * 2;
}
size_t greedy_count_words32(const PimHipRnntPlan* plan) { return (size_t)plan->blocks * kRnntSeenStride + kRnntSeenStride; }

int destroy_rnnt_plan_locked(PimHipRnntPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    int prev = -1;
    hipGetDevice(&prev);
    hipSetDevice(plan->device);
    hipDeviceSynchronize();
    if (plan->bsum) hipFree(plan->bsum);
    if (plan->hx) hipFree(plan->hx);
    if (plan->g_counter) hipFree(plan->g_counter);
    if (plan->greedy) hipFree(plan->greedy);
    if (plan->abort_flag) hipFree(plan->abort_flag);
    if (plan->abort_host) hipHostFree(plan->abort_host);
    if (prev >= 0) hipSetDevice(prev);
    for (size_t i = 0; i < g_rnnt_plans.size(); ++i) {
        if (g_rnnt_plans[i] == plan) {
            g_rnnt_plans.erase(g_rnnt_plans.begin() + i);
            break;
        }
    }
    delete plan;
    return PIMHIP_OK;
}

bool overlap(const void* a, size_t na, const void* b, size_t nb)
{
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + nb && b0 < a0 + na;
}
}  // namespace

namespace pimhip
{
void destroy_all_rnnt_plans_locked()
{
    while (!g_rnnt_plans.empty()) destroy_rnnt_plan_locked(g_rnnt_plans.back());
}
}  // namespace pimhip

extern "C" int pimhip_rnnt_plan_create(PimHipRnntPlan** plan_out, const void* const* params, int n_params, int has_biases, int num_layers,
                                       int64_t input_size, int64_t hidden_size, const void* joint_w1, const void* joint_b1,
                                       int64_t joint_size, int64_t enc_size, const void* joint_w2, const void* joint_b2, int64_t vocab,
                                       void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan_out || !params || !joint_w1 || !joint_w2) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan, params, joint_w1 and joint_w2 must be non-null");
    if (num_layers < 1 || num_layers > kRnntMaxLayers) return fail(PIMHIP_ERR_UNSUPPORTED, "num_layers=%d not in [1, %d]", num_layers, kRnntMaxLayers);
    const int per_layer = has_biases ? 4 : 2;
    if (n_params != per_layer * num_layers)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "%d parameters for %d layers %s biases (expected %d)", n_params, num_layers,
                    has_biases ? "with" : "without", per_layer * num_layers);
    if (hidden_size < 8 || hidden_size > kRnntMaxH || (hidden_size & 7) || input_size < 8 || input_size > kRnntMaxIn || (input_size & 7))
        return fail(PIMHIP_ERR_UNSUPPORTED, "the one-launch step takes hidden_size in [8, %d] and input_size in [8, %d], multiples of 8 (got %lld, %lld)",
                    kRnntMaxH, kRnntMaxIn, (long long)hidden_size, (long long)input_size);
    if (enc_size < 8 || enc_size > kRnntMaxEnc || (enc_size & 7) || joint_size < 8 || joint_size > kRnntMaxJoint || (joint_size & 7) || vocab < 1)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the one-launch step takes enc_size in [8, %d] and joint_size in [8, %d], multiples of 8, and vocab >= 1 "
                                            "(got %lld, %lld, %lld)", kRnntMaxEnc, kRnntMaxJoint, (long long)enc_size, (long long)joint_size, (long long)vocab);
    const int64_t blocks = num_layers * (hidden_size / 8) + joint_size / 8 + (vocab + 7) / 8;
    if (blocks > kRnntMaxBlocks)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the step would need %lld workgroups (one per eight hidden units, joint units and symbols), more than %d: "
                                            "use pimhip_lstm_forward and pimhip_execute_gemv_cat2 / pimhip_execute_gemv", (long long)blocks, kRnntMaxBlocks);
    int per_cu = 0;
    PIMHIP_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, rnnt_step_f16_kernel, kRnntThreads, 0));
    if ((int64_t)per_cu * st->num_cus < blocks)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the %lld workgroups of the one-launch step cannot all be resident on this device", (long long)blocks);
    for (int i = 0; i < n_params; ++i) {
        if (!params[i]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "params[%d] is null", i);
        if (i % per_layer < 2 && !aligned16(params[i])) return fail(PIMHIP_ERR_UNSUPPORTED, "params[%d] must be 16-byte aligned", i);
    }
    if (!aligned16(joint_w1) || !aligned16(joint_w2)) return fail(PIMHIP_ERR_UNSUPPORTED, "joint_w1 and joint_w2 must be 16-byte aligned");

    hipStream_t s = static_cast<hipStream_t>(stream);
    PimHipRnntPlan* plan = new PimHipRnntPlan();
    PIMHIP_HIP_CHECK(hipGetDevice(&plan->device));
    plan->num_layers = num_layers;
    plan->input_size = input_size;
    plan->hidden = hidden_size;
    plan->enc_size = enc_size;
    plan->joint_size = joint_size;
    plan->vocab = vocab;
    plan->w1 = (const half_t*)joint_w1;
    plan->b1 = (const half_t*)joint_b1;
    plan->w2 = (const half_t*)joint_w2;
    plan->b2 = (const half_t*)joint_b2;
    plan->blocks = (int)blocks;
    for (int l = 0; l < num_layers; ++l) {
        plan->w_ih[l] = (const half_t*)params[l * per_layer];
        plan->w_hh[l] = (const half_t*)params[l * per_layer + 1];
    }
    auto cleanup_fail = [&](int status) {
        std::lock_guard<std::mutex> lock(g_mutex);
        destroy_rnnt_plan_locked(plan);
        return status;
    };
#define RNNT_HIP_CHECK(expr)                                                                                    \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) return cleanup_fail(fail(PIMHIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_))); \
    } while (0)
    const int n4 = (int)(4 * hidden_size);
    if (has_biases) {
        RNNT_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->bsum), sizeof(float) * (size_t)num_layers * n4));
        for (int l = 0; l < num_layers; ++l)
            launch_lstm_bias_sum((const half_t*)params[l * 4 + 2], (const half_t*)params[l * 4 + 3], plan->bsum + (size_t)l * n4, n4, s);
    }
    RNNT_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->hx), exchange_words32(plan) * sizeof(unsigned int)));
    launch_fill_u32(reinterpret_cast<unsigned int*>(plan->hx), exchange_words32(plan), ~0u, s);
    RNNT_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->g_counter), sizeof(unsigned int) * (size_t)plan->blocks * kRnntCounterStride));
    launch_fill_u32(plan->g_counter, (size_t)plan->blocks * kRnntCounterStride, 0u, s);
    RNNT_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->greedy), sizeof(unsigned int) * (greedy_exchange_words32(plan) + greedy_count_words32(plan))));
    {
        int greedy_per_cu = 0;
        RNNT_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&greedy_per_cu, rnnt_greedy_f16_kernel, kRnntThreads, 0));
        plan->greedy_resident = (int64_t)greedy_per_cu * st->num_cus >= blocks;
    }
    RNNT_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&plan->abort_flag), sizeof(unsigned int)));
    launch_fill_u32(plan->abort_flag, 1, 0u, s);
    RNNT_HIP_CHECK(hipGetLastError());
    RNNT_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&plan->abort_host), sizeof(unsigned int), hipHostMallocMapped));
    *plan->abort_host = 0u;
    RNNT_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&plan->abort_host_dev), plan->abort_host, 0));
    RNNT_HIP_CHECK(hipStreamSynchronize(s));
#undef RNNT_HIP_CHECK
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        g_rnnt_plans.push_back(plan);
    }
    *plan_out = plan;
    return PIMHIP_OK;
}

extern "C" int pimhip_rnnt_plan_destroy(PimHipRnntPlan* plan)
{
    if (!plan) return PIMHIP_OK;
    std::lock_guard<std::mutex> lock(g_mutex);
    bool known = false;
    for (PimHipRnntPlan* q : g_rnnt_plans) known = known || (q == plan);
    if (!known) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "unknown or already destroyed transducer plan");
    return destroy_rnnt_plan_locked(plan);
}

extern "C" int pimhip_rnnt_plan_set_spin_limit(PimHipRnntPlan* plan, unsigned int spin_limit)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    plan->spin_limit = spin_limit;
    return PIMHIP_OK;
}

extern "C" int pimhip_rnnt_plan_fallbacks(PimHipRnntPlan* plan, uint64_t* events, int* exchanging)
{
    if (!plan || !events) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and events must be non-null");
    *events = plan->gave_up_events + (*plan->abort_host != 0u ? 1u : 0u);
    if (exchanging) *exchanging = (plan->alone || *events >= kRnntEventsBeforeAlone) ? 0 : 1;
    return PIMHIP_OK;
}

extern "C" int pimhip_rnnt_step(PimHipRnntPlan* plan, const void* x, const void* h_prev, const void* c_prev, const void* f, void* hn,
                                void* cn, void* logits, void* joint_hidden, int run_prediction, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!h_prev || !f || !logits) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "h_prev, f and logits must be non-null");
    if (!aligned16(h_prev) || !aligned16(f)) return fail(PIMHIP_ERR_UNSUPPORTED, "h_prev and f must be 16-byte aligned");
    const size_t state_bytes = sizeof(half_t) * (size_t)plan->num_layers * plan->hidden;
    if (run_prediction) {
        if (!x || !c_prev || !hn || !cn) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "x, c_prev, hn and cn must be non-null when the prediction network runs");
        if (!aligned16(x)) return fail(PIMHIP_ERR_UNSUPPORTED, "x must be 16-byte aligned");
        // A block whose wait gives up recomputes from the step's inputs: they have to stay what they were.
        if (overlap(hn, state_bytes, h_prev, state_bytes) || overlap(hn, state_bytes, c_prev, state_bytes) ||
            overlap(cn, state_bytes, h_prev, state_bytes) || overlap(cn, state_bytes, c_prev, state_bytes))
            return fail(PIMHIP_ERR_INVALID_ARGUMENT, "hn / cn must not overlap h_prev / c_prev (keep two state buffers and swap them)");
    }

    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (*plan->abort_host != 0u && !capturing) {
        // A wait of an earlier launch gave up.  That step's result was completed by the blocks themselves, and every step
        // since has run self-sufficient (the abort word stays up on the device); here, outside any capture, the exchange is
        // put back in order: drain the stream (steps sharing a plan are ordered on one stream), refill the entries, clear
        // the words.  A plan that has needed this kRnntEventsBeforeAlone times stops exchanging for good.
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        *plan->abort_host = 0u;
        ++plan->gave_up_events;
        if (plan->gave_up_events >= kRnntEventsBeforeAlone) plan->alone = true;
        launch_fill_u32(reinterpret_cast<unsigned int*>(plan->hx), exchange_words32(plan), ~0u, s);
        launch_fill_u32(plan->g_counter, (size_t)plan->blocks * kRnntCounterStride, 0u, s);
        launch_fill_u32(plan->abort_flag, 1, 0u, s);
        PIMHIP_HIP_CHECK(hipGetLastError());
    }
    RnntStepArgs a;
    memset(&a, 0, sizeof(a));
    const int n4 = (int)(4 * plan->hidden);
    for (int l = 0; l < plan->num_layers; ++l) {
        a.layer[l].w_ih = plan->w_ih[l];
        a.layer[l].w_hh = plan->w_hh[l];
        a.layer[l].bsum = plan->bsum ? plan->bsum + (size_t)l * n4 : nullptr;
        a.layer[l].in_w = (int)(l == 0 ? plan->input_size : plan->hidden);
    }
    a.hn = (half_t*)hn;
    a.cn = (half_t*)cn;
    a.logits = (half_t*)logits;
    a.joint_hidden = (half_t*)joint_hidden;
    a.w1 = plan->w1;
    a.b1 = plan->b1;
    a.w2 = plan->w2;
    a.b2 = plan->b2;
    a.hx = plan->hx;
    a.g_counter = plan->g_counter;
    a.abort_flag = plan->abort_flag;
    a.abort_host = plan->abort_host_dev;
    a.F = (int)plan->enc_size;
    a.V = (int)plan->vocab;
    a.spin_limit = plan->spin_limit;
    a.alone = plan->alone ? 1 : 0;
    // All blocks have to be resident at once, like the sequence kernel's: ordered after it on other streams.
    if (!capturing) {
        rc = order_after_previous_sequence_launch(st, s);
        if (rc != PIMHIP_OK) return rc;
    }
    rnnt_step_f16_kernel<<<dim3((unsigned)plan->blocks), dim3(kRnntThreads), 0, s>>>(
        (const half_t*)x, (const half_t*)h_prev, (const half_t*)c_prev, (const half_t*)f, plan->num_layers, (int)plan->hidden,
        (int)plan->joint_size, run_prediction ? 1 : 0, a);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}

extern "C" int pimhip_rnnt_greedy_decode(PimHipRnntPlan* plan, const void* enc, int64_t n_frames, const void* embedding,
                                         int64_t embedding_rows, const void* x0, const void* h0, const void* c0, int run_prediction_first,
                                         int blank, int max_symbols_per_frame, int64_t max_symbols, int32_t* symbols, int32_t* result,
                                         void* hn, void* cn, void* stream)
{
    DeviceState* st = nullptr;
    int rc = current_device_state(&st);
    if (rc != PIMHIP_OK) return rc;
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    int dev = -1;
    PIMHIP_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan belongs to device %d, current device is %d", plan->device, dev);
    if (!embedding || !result || (!enc && n_frames > 0) || (!symbols && max_symbols > 0))
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "enc, embedding, symbols and result must be non-null");
    if (n_frames < 0 || n_frames > INT32_MAX || max_symbols < 0 || max_symbols > INT32_MAX || max_symbols_per_frame < 1)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "n_frames=%lld, max_symbols=%lld, max_symbols_per_frame=%d", (long long)n_frames,
                    (long long)max_symbols, max_symbols_per_frame);
    if (plan->vocab > kRnntGreedyMaxVocab)
        return fail(PIMHIP_ERR_UNSUPPORTED, "the one-launch loop takes up to %d symbols (the plan has %lld): drive pimhip_rnnt_step from the host",
                    kRnntGreedyMaxVocab, (long long)plan->vocab);
    if (blank < 0 || blank >= plan->vocab) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "blank=%d not in [0, %lld)", blank, (long long)plan->vocab);
    if (embedding_rows < plan->vocab)
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "embedding has %lld rows, the joint network emits %lld symbols", (long long)embedding_rows,
                    (long long)plan->vocab);
    if (run_prediction_first && !x0) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "x0 must be non-null when the first step runs the prediction network");
    if (!aligned16(enc) || !aligned16(embedding) || !aligned16(x0) || !aligned16(h0))
        return fail(PIMHIP_ERR_UNSUPPORTED, "enc, embedding, x0 and h0 must be 16-byte aligned");
    const size_t state_bytes = sizeof(half_t) * (size_t)plan->num_layers * plan->hidden;
    // A workgroup that has to decode alone starts again from h0 / c0.
    if ((hn && h0 && overlap(hn, state_bytes, h0, state_bytes)) || (hn && c0 && overlap(hn, state_bytes, c0, state_bytes)) ||
        (cn && h0 && overlap(cn, state_bytes, h0, state_bytes)) || (cn && c0 && overlap(cn, state_bytes, c0, state_bytes)))
        return fail(PIMHIP_ERR_INVALID_ARGUMENT, "hn / cn must not overlap h0 / c0");

    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    if (*plan->abort_host != 0u && !capturing) {
        // as in pimhip_rnnt_step: a wait of an earlier launch gave up (its result was completed all the same)
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        *plan->abort_host = 0u;
        ++plan->gave_up_events;
        if (plan->gave_up_events >= kRnntEventsBeforeAlone) plan->alone = true;
        launch_fill_u32(reinterpret_cast<unsigned int*>(plan->hx), exchange_words32(plan), ~0u, s);
        launch_fill_u32(plan->g_counter, (size_t)plan->blocks * kRnntCounterStride, 0u, s);
        launch_fill_u32(plan->abort_flag, 1, 0u, s);
        PIMHIP_HIP_CHECK(hipGetLastError());
    }
    RnntGreedyArgs a;
    memset(&a, 0, sizeof(a));
    const int n4 = (int)(4 * plan->hidden);
    for (int l = 0; l < plan->num_layers; ++l) {
        a.layer[l].w_ih = plan->w_ih[l];
        a.layer[l].w_hh = plan->w_hh[l];
        a.layer[l].bsum = plan->bsum ? plan->bsum + (size_t)l * n4 : nullptr;
        a.layer[l].in_w = (int)(l == 0 ? plan->input_size : plan->hidden);
    }
    a.w1 = plan->w1;
    a.b1 = plan->b1;
    a.w2 = plan->w2;
    a.b2 = plan->b2;
    a.enc = (const half_t*)enc;
    a.embedding = (const half_t*)embedding;
    a.x0 = (const half_t*)x0;
    a.h0 = (const half_t*)h0;
    a.c0 = (const half_t*)c0;
    a.hn = (half_t*)hn;
    a.cn = (half_t*)cn;
    a.symbols = symbols;
    a.result = result;
    a.hx = reinterpret_cast<unsigned long long*>(plan->greedy);
    a.seen = plan->greedy + greedy_exchange_words32(plan);
    a.solo_owner = a.seen + (size_t)plan->blocks * kRnntSeenStride;
    a.abort_flag = plan->abort_flag;
    a.abort_host = plan->abort_host_dev;
    a.L = plan->num_layers;
    a.H = (int)plan->hidden;
    a.F = (int)plan->enc_size;
    a.J = (int)plan->joint_size;
    a.V = (int)plan->vocab;
    a.T = (int)n_frames;
    a.emb_rows = (int)embedding_rows;
    a.emb_in_lds = (embedding_rows + 1) * plan->input_size <= kRnntGreedyEmbHalfs ? 1 : 0;
    a.blank = blank;
    a.max_symbols = (int)max_symbols;
    a.max_per_frame = max_symbols_per_frame;
    a.run_pred_first = run_prediction_first ? 1 : 0;
    a.spin_limit = plan->spin_limit;
    a.alone = (plan->alone || !plan->greedy_resident) ? 1 : 0;
    if (!capturing) {
        rc = order_after_previous_sequence_launch(st, s);
        if (rc != PIMHIP_OK) return rc;
    }
    // fill kernels, not memsets: the call can be recorded into a HIP graph
    launch_fill_u32(plan->greedy, greedy_exchange_words32(plan), ~0u, s);
    launch_fill_u32(plan->greedy + greedy_exchange_words32(plan), greedy_count_words32(plan), 0u, s);
    rnnt_greedy_f16_kernel<<<dim3(a.alone ? 1u : (unsigned)plan->blocks), dim3(kRnntThreads), 0, s>>>(a);
    PIMHIP_HIP_CHECK(hipGetLastError());
    return PIMHIP_OK;
}
