// The LSTM part of the C ABI (include/pimhip.h): plans, the choice between the step kernel and the persistent sequence
// kernels, and their launches.
#include "api_common.h"
#include "../../include/pimhip_probe.h"
#include "lstm_kernels.h"
#include "lstm_xcd_kernels.h"

using namespace pimhip;

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
    // Waits of the persistent kernels that gave up, as far as the host has seen them (pimhip_lstm_plan_fallbacks).  Such a
    // forward is completed by the workgroups themselves; after kLstmEventsBeforeSafe events the plan stops choosing
    // kernels whose workgroups wait for one another.
    unsigned long long gave_up_events = 0;
    bool safe_only = false;
    // Automatic mode: the kernel family measured fastest on this plan for sequence lengths in [2^b, 2^(b+1)), 0 = not
    // measured yet (pimhip_lstm_forward measures on the first eager call of a bucket; see measured_mode below).
    unsigned char measured_mode[32] = {};
    bool measure = true;             // pimhip_lstm_plan_set_measure
    hipEvent_t tune_event[2] = {nullptr, nullptr};
};

namespace
{
constexpr unsigned long long kLstmEventsBeforeSafe = 3;
}

namespace
{
std::vector<PimHipLstmPlan*> g_plans;

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
    for (hipEvent_t e : plan->tune_event)
        if (e) hipEventDestroy(e);
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

namespace pimhip
{
void destroy_all_lstm_plans_locked()
{
    while (!g_plans.empty()) destroy_plan_locked(g_plans.back());
}
}  // namespace pimhip

namespace
{
__global__ void xcc_map_kernel(unsigned int* out)
{
    if (threadIdx.x == 0) out[blockIdx.x] = hw_xcc_id();
}

// The per-XCD kernel finds its place by the hardware's XCC_ID and relies on two things the hardware does today: ids 0..7,
// and workgroup b of a launch going to XCD (b + o) % 8 for some start o.  One probe launch of the same grid tells whether
// this device, as this process sees it (CU masks, partition mode), behaves so; where it does not, the kernel is not offered.
int xcd_dispatch_is_a_rotation(int blocks, hipStream_t s, bool* ok)
{
    *ok = false;
    unsigned int* dev_map = nullptr;
    PIMHIP_HIP_CHECK(hipMalloc(&dev_map, (size_t)blocks * sizeof(unsigned int)));
    xcc_map_kernel<<<(unsigned)blocks, kXcdThreads, 0, s>>>(dev_map);
    std::vector<unsigned int> map((size_t)blocks, 0u);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(map.data(), dev_map, (size_t)blocks * sizeof(unsigned int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    hipFree(dev_map);
    if (e != hipSuccess) return fail(PIMHIP_ERR_HIP, "probing the placement of workgroups failed: %s", hipGetErrorString(e));
    bool rotation = map[0] < (unsigned)kXcdCount;
    for (int b = 1; rotation && b < blocks; ++b) rotation = map[(size_t)b] == (map[0] + (unsigned)b) % kXcdCount;
    *ok = rotation;
    return PIMHIP_OK;
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
            launch_lstm_bias_sum(c.b_ih, c.b_hh, c.bsum, (int)(4 * H), s);
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
            launch_pack_w_fragments(c.w_ih, c.w_ih_packed, 4 * H, c.in_w, ntiles, c.ksteps, s);
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
        launch_fill_u32(plan->g_counters, kSeqMaxChains + 1, 2u, s);
        PLAN_HIP_CHECK(hipGetLastError());
    }
    // One recurrence per XCD: the part this is written for has 8 XCDs of 32 CUs, a group is one workgroup per CU of one.
    if (H <= kXcdMaxH && plan->num_cus == kXcdCount * kXcdMembers) {
        int per_cu = 0;
        int per_cu_pipe = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lstm_xcd_f16_kernel<false>, kXcdThreads, 0));
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_pipe, lstm_xcd_f16_kernel<true>, kXcdThreads, 0));
        plan->xcd_ok = per_cu >= 1 && per_cu_pipe >= 1;
        if (plan->xcd_ok) {
            bool rotation = false;
            const int rc_probe = xcd_dispatch_is_a_rotation(kXcdCount * kXcdMembers, s, &rotation);
            if (rc_probe != PIMHIP_OK) return cleanup_fail(rc_probe);
            plan->xcd_ok = rotation;
        }
        int per_cu_res = 0;
        PLAN_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_res, lstm_xcd_res_f16_kernel, kXcdThreads, 0));
        plan->xcd_res_ok = plan->xcd_ok && per_cu_res >= 1;
    }
    if (plan->xcd_ok) {
        const size_t words = (size_t)kXcdRegionWords * kXcdMaxChains;
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_hx, words * sizeof(unsigned int)));
        launch_fill_u32(plan->xcd_hx, words, 0u, s);
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_g_counters, kXcdMaxChains * sizeof(unsigned int)));
        launch_fill_u32(plan->xcd_g_counters, kXcdMaxChains, 2u, s);
        PLAN_HIP_CHECK(hipMalloc(&plan->xcd_claims, kXcdCount * kXcdMembers * sizeof(unsigned int)));
        launch_fill_u32(plan->xcd_claims, kXcdCount * kXcdMembers, 0u, s);
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
    if (plan->first_residual_layer != first_residual_layer) memset(plan->measured_mode, 0, sizeof(plan->measured_mode));
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
    if (*plan->abort_host == 2u) {
        // The one event that leaves a forward undefined: two workgroups of the per-XCD kernel with the same rank on one XCD
        // (some units then belong to nobody).  Reported once, here or by the next pimhip_lstm_forward.  The caller has
        // synchronised the stream, so the kernel that set the word has ended.
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        return xcd_placement_failure(plan);
    }
    // A wait that gave up is no error: the workgroups completed that forward by themselves (pimhip_lstm_plan_fallbacks
    // counts such events; the next forward outside a capture re-initialises the exchange).
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_fallbacks(PimHipLstmPlan* plan, uint64_t* events, int* exchanging)
{
    if (!plan || !events) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and events must be non-null");
    *events = plan->gave_up_events + (*plan->abort_host == 1u ? 1u : 0u);
    if (exchanging) *exchanging = (plan->safe_only || *events >= kLstmEventsBeforeSafe) ? 0 : 1;
    return PIMHIP_OK;
}

namespace
{
int measure_modes(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y, void* hn, void* cn,
                  int64_t seq_len, void* stream, int bucket, bool xcd_takes_it, bool seq_takes_it);

// pimhip_lstm_forward with the plan's mode replaced by `forced_mode` when that is not negative (the measurement of
// automatic mode runs the call under every kernel family that takes it).
int lstm_forward_impl(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y, void* hn, void* cn,
                      int64_t seq_len, void* stream, int forced_mode)
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

    // Whether `s` is recording a graph matters only to the sequence kernels and to the recovery paths: a call of one step,
    // the per-token call of a decoding loop, does not pay for the query.
    bool capturing = false;
    if (T >= 2 || *plan->abort_host != 0u) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        PIMHIP_HIP_CHECK(hipStreamIsCapturing(s, &capture));
        capturing = capture != hipStreamCaptureStatusNone;
    }
    if (*plan->abort_host != 0u && !capturing) {
        // A wait of an earlier sequence kernel of this plan gave up.  That forward was completed by the workgroups
        // themselves and every sequence launch since has run self-sufficient (the abort word stays up on the device); here,
        // outside any capture, the exchange is put back in order.  The word is cleared only after the stream has drained
        // (calls sharing a plan are ordered on one stream), so that no kernel sets it again.
        PIMHIP_HIP_CHECK(hipStreamSynchronize(s));
        const bool misplaced = *plan->abort_host == 2u;
        *plan->abort_host = 0u;
        plan->reset_exchange = true;
        if (misplaced) return xcd_placement_failure(plan);  // (the one event that leaves a forward undefined)
        if (++plan->gave_up_events >= kLstmEventsBeforeSafe) plan->safe_only = true;
    }
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
    // (a plan whose waits have given up kLstmEventsBeforeSafe times runs one launch per step from then on: no workgroup of
    // those kernels waits for another)
    const bool xcd_takes_it = T >= 2 && T <= kSeqMaxT - 2 && plan->xcd_ok && !res_pipeline_missing && !plan->safe_only;
    const bool seq_takes_it = T >= 2 && T + kSeqMaxChains <= kSeqMaxT && plan->seq_kernel_ok && !plan->safe_only;
    int mode = forced_mode >= 0 ? forced_mode : plan->mode;
    if (mode == 0 && T >= 2) {
        // Automatic: what was measured fastest on this plan for sequences of about this length; failing that (nothing
        // measured yet and no way to measure now) the thresholds above.
        int bucket = 0;
        while ((T >> (bucket + 1)) != 0 && bucket < 31) ++bucket;
        if (plan->measured_mode[bucket] == 0 && plan->measure && !capturing && forced_mode < 0 && (xcd_takes_it || seq_takes_it)) {
            rc = measure_modes(plan, x, h0, c0, y, hn, cn, seq_len, stream, bucket, xcd_takes_it, seq_takes_it);
            if (rc != PIMHIP_OK) return rc;
            return PIMHIP_OK;  // (the last of the measured runs was the call, under the mode that won)
        }
        if (plan->measured_mode[bucket] != 0) mode = plan->measured_mode[bucket];
    }
    const bool use_xcd = xcd_takes_it && (mode == 4 || (mode == 0 && xcd_pays));
    const bool use_seq = !use_xcd && T >= 2 && T + kSeqMaxChains <= kSeqMaxT && !plan->safe_only &&
                         (mode == 2 || mode == 3 || (mode == 0 && plan->seq_kernel_ok));
    if (use_seq && !plan->seq_kernel_ok) return fail(PIMHIP_ERR_UNSUPPORTED, "persistent sequence kernel not available for this plan");
    if ((use_seq || use_xcd) && plan->reset_exchange) {
        // After a time-out or a change of the entry layout: re-arm the flag and bring the exchange buffer and its step
        // counters back to their initial state.
        if (capturing)
            return fail(PIMHIP_ERR_UNSUPPORTED, "the plan's exchange buffer has to be re-initialised (after a change of mode), which a "
                                                "graph must not record: run one forward outside the capture first");
        launch_fill_u32(plan->abort_flag, 1, 0u, s);
        if (plan->hx) {
            const size_t words = plan->hx_region_words * kSeqMaxChains;
            launch_fill_u32(plan->hx, words, 0u, s);
            launch_fill_u32(plan->g_counters, kSeqMaxChains + 1, 2u, s);
        }
        if (plan->xcd_hx) {
            const size_t words = (size_t)kXcdRegionWords * kXcdMaxChains;
            launch_fill_u32(plan->xcd_hx, words, 0u, s);
            launch_fill_u32(plan->xcd_g_counters, kXcdMaxChains, 2u, s);
            launch_fill_u32(plan->xcd_claims, kXcdCount * kXcdMembers, 0u, s);
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
        launch_add_f16_vec(out, in, out, (long)T * H / 8, (long)(H / 8), 0, st->num_cus, s);
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
            // the first layer's projection, and beside it (blocks of the same launch) the hand-over slots marked empty
            float* outs1[1] = {plan->xproj};
            const float* bs1[1] = {cf.bsum};
            if (cf.w_ih_packed) {
                const half_t* ws1[1] = {cf.w_ih_packed};
                rc = launch_input_projection_packed(1, outs1, layer_in, ws1, bs1, T, cf.in_w, 4 * H, cf.ksteps, s, &seg, 2 * (n - 1));
            } else {
                const half_t* ws1[1] = {cf.w_ih};
                rc = launch_input_projection(1, outs1, layer_in, ws1, bs1, T, cf.in_w, 4 * H, s);
                launch_fill_segments(seg, 2 * (n - 1), 0xffffffffu, s);
            }
            if (rc != PIMHIP_OK) return rc;
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
                        if (plan->seq_units8_ok && mode != 3)
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
                    float* outs1[1] = {xp};
                    const half_t* ws1[1] = {c.w_ih};
                    const float* bs1[1] = {c.bsum};
                    rc = launch_input_projection(1, outs1, layer_in, ws1, bs1, T, in_w, 4 * H, s);
                    if (rc != PIMHIP_OK) return rc;
                }
                float* cst = plan->c_state + (size_t)d * H;
                const unsigned grid = (unsigned)((H + 3) / 4);
                // what a step's launch reads: W_hh, and W_ih when the projection is made in the same kernel
                const int keep = (unsigned long long)(4 * H) * (unsigned long long)(H + (fuse_xproj ? in_w : 0)) * sizeof(half_t) <= kKeepCachedBytes;
                for (int64_t step = 0; step < T; ++step) {
                    const int64_t t = d ? (T - 1 - step) : step;
                    const int64_t tp = d ? (t + 1) : (t - 1);
                    const half_t* h_prev = (step == 0) ? h0c : (yd + tp * y_stride);
                    const bool last = step == T - 1;
                    (keep ? lstm_step_f16_kernel<4, true> : lstm_step_f16_kernel<4, false>)<<<grid, 256, 0, s>>>(
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

// Runs the call once under every kernel family that takes it and keeps, for sequence lengths of this bucket, the fastest:
// the counterpart of the reference timing both of its libraries on the first inference and keeping the faster per layer
// (runtime/source/executor/stream_executor.cpp:312-339).  Every run computes the same call into the same outputs; the last
// one is made under the winner, so the caller gets that mode's bits.  Synchronises `stream` (HIP events).
int measure_modes(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y, void* hn, void* cn,
                  int64_t seq_len, void* stream, int bucket, bool xcd_takes_it, bool seq_takes_it)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (hipEvent_t& e : plan->tune_event)
        if (!e) PIMHIP_HIP_CHECK(hipEventCreate(&e));
    int candidates[3], n = 0;
    if (xcd_takes_it) candidates[n++] = 4;
    if (seq_takes_it) candidates[n++] = 2;
    if (seq_len <= 8) candidates[n++] = 1;  // (one launch per step only ever wins on the shortest sequences)
    int best = candidates[0];
    float best_ms = -1.0f;
    const unsigned long long events_before = plan->gave_up_events;
    for (int i = 0; i < n && n > 1; ++i) {
        float ms_min = -1.0f;
        for (int rep = 0; rep < 3; ++rep) {  // the first run of a mode also loads its code and warms the weights
            PIMHIP_HIP_CHECK(hipEventRecord(plan->tune_event[0], s));
            const int rc = lstm_forward_impl(plan, x, h0, c0, y, hn, cn, seq_len, stream, candidates[i]);
            if (rc != PIMHIP_OK) return rc;
            PIMHIP_HIP_CHECK(hipEventRecord(plan->tune_event[1], s));
            PIMHIP_HIP_CHECK(hipEventSynchronize(plan->tune_event[1]));
            float ms = 0.0f;
            PIMHIP_HIP_CHECK(hipEventElapsedTime(&ms, plan->tune_event[0], plan->tune_event[1]));
            if (rep > 0 && (ms_min < 0.0f || ms < ms_min)) ms_min = ms;
        }
        // (a mode in which a wait gave up while it was measured is not a candidate)
        const bool gave_up = *plan->abort_host != 0u || plan->gave_up_events != events_before;
        if (!gave_up && (best_ms < 0.0f || ms_min < best_ms)) {
            best_ms = ms_min;
            best = candidates[i];
        }
    }
    plan->measured_mode[bucket] = (unsigned char)best;
    return lstm_forward_impl(plan, x, h0, c0, y, hn, cn, seq_len, stream, best);
}
}  // namespace

extern "C" int pimhip_lstm_forward(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y,
                                   void* hn, void* cn, int64_t seq_len, void* stream)
{
    return lstm_forward_impl(plan, x, h0, c0, y, hn, cn, seq_len, stream, -1);
}

extern "C" int pimhip_lstm_plan_set_measure(PimHipLstmPlan* plan, int enabled)
{
    if (!plan) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan is null");
    plan->measure = enabled != 0;
    if (!plan->measure) memset(plan->measured_mode, 0, sizeof(plan->measured_mode));
    return PIMHIP_OK;
}

extern "C" int pimhip_lstm_plan_measured_mode(PimHipLstmPlan* plan, int64_t seq_len, int* mode)
{
    if (!plan || !mode) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "plan and mode must be non-null");
    if (seq_len < 2) return fail(PIMHIP_ERR_INVALID_ARGUMENT, "seq_len=%lld: one step has one kernel", (long long)seq_len);
    int bucket = 0;
    while ((seq_len >> (bucket + 1)) != 0 && bucket < 31) ++bucket;
    *mode = plan->measured_mode[bucket];
    return PIMHIP_OK;
}
