// The decoder step of the C ABI (include/pimhip.h): a stack of seq_len-1 LSTM cells, the attention context, the residual
// sums and the classifier in one persistent launch.
#include "api_common.h"
#include "decoder_kernels.h"

#include <algorithm>

using namespace pimhip;

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
    unsigned int* hx = nullptr;       // [kDecStages][blocks][kDecEntryWords], zeros before the first launch
    // One allocation behind `notes`: the blocks' notes (kDecNoteWords 64-bit words each, and one word more; zeros before the
    // first launch), then the parked h and c ([num_layers][H] fp16 each).
    unsigned long long* notes = nullptr;
    half_t* parked_h = nullptr;
    half_t* parked_c = nullptr;
    unsigned int* abort_host = nullptr;
    unsigned int* abort_host_dev = nullptr;
    unsigned int spin_limit = 1u << 22;
    unsigned long long gave_up_events = 0;  // waits that gave up, as far as the host has seen them (pimhip_decoder_plan_fallbacks)
    int blocks = 0;
};

namespace
{
std::vector<PimHipDecoderPlan*> g_decoder_plans;
constexpr unsigned long long kDecEventsBeforeImpatient = 3;  // waits given up before every wait of a plan's steps is short

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
    if (plan->notes) hipFree(plan->notes);
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

namespace pimhip
{
void destroy_all_decoder_plans_locked()
{
    while (!g_decoder_plans.empty()) destroy_decoder_plan_locked(g_decoder_plans.back());
}
}  // namespace pimhip

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
        launch_lstm_bias_sum(has_biases ? (const half_t*)q[2] : nullptr, has_biases ? (const half_t*)q[3] : nullptr,
                             plan->bsum + (size_t)l * 4 * H, (int)(4 * H), s);
    }
    DEC_HIP_CHECK(hipGetLastError());
    const size_t words = (size_t)kDecStages * blocks * kDecEntryWords;
    DEC_HIP_CHECK(hipMalloc(&plan->hx, words * sizeof(unsigned int)));
    launch_fill_u32(plan->hx, words, 0u, s);
    {
        const size_t note_words = 2 * ((size_t)blocks * kDecNoteWords + 1);                  // 32-bit words
        const size_t state_words = ((size_t)num_layers * H * sizeof(half_t) + 3) / 4;         // per parked array
        const size_t aux_words = note_words + 2 * state_words;
        DEC_HIP_CHECK(hipMalloc(&plan->notes, aux_words * sizeof(unsigned int)));
        unsigned int* aux = reinterpret_cast<unsigned int*>(plan->notes);
        plan->parked_h = reinterpret_cast<half_t*>(aux + note_words);
        plan->parked_c = reinterpret_cast<half_t*>(aux + note_words + state_words);
        launch_fill_u32(aux, aux_words, 0u, s);
    }
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
    // A wait that gives up is made good inside the same launch (the entries that did not come are computed where they are
    // missed), so there is nothing to report as an error.  pimhip_decoder_plan_fallbacks counts the events.
    return PIMHIP_OK;
}

extern "C" int pimhip_decoder_plan_fallbacks(PimHipDecoderPlan* plan, uint64_t* events, int* patient)
{
    if (!plan || !events) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and events must be non-null");
    *events = plan->gave_up_events + (*plan->abort_host != 0u ? 1u : 0u);
    if (patient) *patient = *events >= kDecEventsBeforeImpatient ? 0 : 1;
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
    if (*plan->abort_host != 0u && !capturing) {
        // A wait gave up in an earlier step; that step made the missing entries itself and its results stand.  The exchange
        // buffer needs nothing (every block has written every entry of that launch by the time it ended).
        *plan->abort_host = 0u;
        ++plan->gave_up_events;
    }
    // A plan whose steps have had to do that kDecEventsBeforeImpatient times keeps every wait short: a step then costs a
    // few milliseconds at worst when part of the grid is kept from running, instead of a second.
    const unsigned int spin_limit = plan->gave_up_events >= kDecEventsBeforeImpatient ? std::min(plan->spin_limit, kDecImpatientPolls) : plan->spin_limit;

    DecoderStepArgs a;
    memset(&a, 0, sizeof(a));
    a.n_layers = L;
    for (int l = 0; l < L; ++l) {
        if (!h_prev[l] || !c_prev[l] || !hn[l] || !cn[l]) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "state pointers of layer %d are null", l);
        if (!aligned16(h_prev[l]) || !aligned16(c_prev[l]))
            return fail(PIMHIP_ERR_UNSUPPORTED, "h_prev and c_prev of layer %d must be 16-byte aligned", l);
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
    a.notes = plan->notes;
    a.parked_h = plan->parked_h;
    a.parked_c = plan->parked_c;
    a.abort_host = plan->abort_host_dev;
    a.spin_limit = spin_limit;
    a.H = (int)H;
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

