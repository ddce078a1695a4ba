// Bodies for the reference's GEMV / LSTM operators on top of libpimhip.so (see aten_ops_pimhip.h).
// Dispatch rules and output shapes follow runtime/source/executor/op_executor/aten_ops.cpp:609-932; the arithmetic is in
// the HIP kernels behind the C ABI.  at::Tensor is used for device memory only.
#include "aten_ops_pimhip.h"

#include <c10/hip/HIPStream.h>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>

#include "../../include/pimhip.h"

namespace nn_compiler
{
namespace runtime
{
namespace utils
{
namespace
{
void check(int rc)
{
    if (rc != PIMHIP_OK) throw NNRuntimeException(std::string("pimhip: ") + pimhip_last_error());
}
}  // namespace

void gemmBroadcast(std::vector<int64_t>& shape1, std::vector<int64_t>& shape2)
{
    int64_t a[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
    int ra = (int)shape1.size(), rb = (int)shape2.size();
    if (ra < 1 || ra > 4 || rb < 1 || rb > 4) throw NNRuntimeException("The dims of input and weight must less than 4");
    for (int i = 0; i < ra; ++i) a[i] = shape1[i];
    for (int i = 0; i < rb; ++i) b[i] = shape2[i];
    const int rc = pimhip_gemm_broadcast(a, &ra, b, &rb);
    if (rc != PIMHIP_OK && rc != PIMHIP_ERR_UNSUPPORTED) check(rc);
    shape1.assign(a, a + ra);
    shape2.assign(b, b + rb);
    if (rc == PIMHIP_ERR_UNSUPPORTED) throw NNRuntimeException(std::string("gemmBroadcast: ") + pimhip_last_error());
}

GEMM_TYPE getGemmType(std::vector<int64_t> self_shape, std::vector<int64_t> other_shape)
{
    if (self_shape.size() != 4 || other_shape.size() != 4) throw NNRuntimeException("getGemmType takes two rank-4 shapes");
    int t = 0;
    check(pimhip_get_gemm_type(self_shape.data(), other_shape.data(), &t));
    switch (t) {
        case PIMHIP_GEMM_VV: return GEMM_TYPE::VV;
        case PIMHIP_GEMM_VM: return GEMM_TYPE::VM;
        case PIMHIP_GEMM_MV: return GEMM_TYPE::MV;
        case PIMHIP_GEMM_MM: return GEMM_TYPE::MM;
        default: return GEMM_TYPE::UNKNOW;
    }
}
}  // namespace utils

namespace op_executor
{
using utils::GEMM_TYPE;
using utils::NNRuntimeException;

namespace
{
void check(int rc)
{
    if (rc != PIMHIP_OK) throw NNRuntimeException(std::string("pimhip: ") + pimhip_last_error());
}

// The stream a call runs on: the caller's, or torch's current stream of the current device when none is given (the
// null stream unless the caller has made another one current), which is the stream the at::Tensor outputs allocated
// here belong to.
void* streamOrCurrent(void* stream) { return stream ? stream : static_cast<void*>(c10::hip::getCurrentHIPStream().stream()); }

void requireHalfOnGpu(const at::Tensor& t, const char* what)
{
    if (!t.defined()) return;
    if (!t.is_cuda()) throw NNRuntimeException(std::string(what) + " must live on the GPU (this path has no CPU fallback)");
    if (t.scalar_type() != at::kHalf) throw NNRuntimeException(std::string(what) + " must be fp16");
}

// The per-token calls of a decoding loop (a 1024 x 1024 product runs 2.5 us on the device) must not cost the host more
// than the kernel takes, so the common case below makes no tensor besides the output: no reshape, no transpose view,
// no shape vectors on the heap.

// The elements of `t` as one dense vector: its own memory when contiguous, else a copy kept alive in `hold`.
const void* denseData(const at::Tensor& t, at::Tensor& hold)
{
    if (t.is_contiguous()) return t.data_ptr();
    hold = t.contiguous();
    return hold.data_ptr();
}

// The last two dims of `w` (every dim before them has size 1) as a matrix of `rows` x `cols` usable without a copy.
// `flipped` is set when its memory is the transpose of a row-major matrix, i.e. the other operand order on the same
// bytes (what SwapAddmmInputs hands over, where the reference calls .contiguous(), aten_ops.cpp:630-632); anything else
// is copied into `hold`.  `ld` is the row pitch of the matrix as it lies in memory.
const void* weightData(const at::Tensor& w, int64_t rows, int64_t cols, bool& flipped, int64_t& ld, at::Tensor& hold)
{
    flipped = false;
    const int64_t d = w.dim();
    const int64_t sr = d >= 2 ? w.stride(d - 2) : cols, sc = w.stride(d - 1);
    if ((sc == 1 || cols == 1) && (rows == 1 || sr >= cols)) {
        ld = rows > 1 ? sr : cols;
        return w.data_ptr();
    }
    if ((sr == 1 || rows == 1) && (cols == 1 || sc >= rows)) {
        flipped = true;
        ld = cols > 1 ? sc : rows;
        return w.data_ptr();
    }
    hold = w.contiguous();
    ld = cols;
    return hold.data_ptr();
}

// out (already allocated, out_w elements) = act(weight . x + bias); weight is [in_w, out_w] for I_X_W, [out_w, in_w] for W_X_I.
void gemvInto(at::Tensor& out, const at::Tensor& x, const at::Tensor& weight, const at::Tensor& bias, int64_t in_w, int64_t out_w,
              int order, int act, void* stream)
{
    at::Tensor hold_x, hold_w, hold_b;
    bool flipped = false;
    int64_t ld = 0;
    const bool mv = order == PIMHIP_W_X_I;
    const void* w = weightData(weight, mv ? out_w : in_w, mv ? in_w : out_w, flipped, ld, hold_w);
    if (flipped) order = mv ? PIMHIP_I_X_W : PIMHIP_W_X_I;
    if (x.numel() != in_w || weight.numel() != in_w * out_w) throw NNRuntimeException("operands do not form a matrix-vector product");
    const void* b = nullptr;
    if (bias.defined()) {
        if (bias.numel() != out_w) throw NNRuntimeException("bias length does not match the GEMV output");
        b = denseData(bias, hold_b);
    }
    check(pimhip_execute_gemv(out.data_ptr(), denseData(x, hold_x), w, b, in_w, out_w, ld, act, order, streamOrCurrent(stream)));
}

// Shape classes of the two operands, by the reference's own rules, on the stack.
GEMM_TYPE classify(const at::Tensor& a, const at::Tensor& b)
{
    int64_t s1[4] = {0, 0, 0, 0}, s2[4] = {0, 0, 0, 0};
    int r1 = (int)a.dim(), r2 = (int)b.dim();
    if (r1 < 1 || r1 > 4 || r2 < 1 || r2 > 4) throw NNRuntimeException("The dims of input and weight must less than 4");
    for (int i = 0; i < r1; ++i) s1[i] = a.size(i);
    for (int i = 0; i < r2; ++i) s2[i] = b.size(i);
    const int rc = pimhip_gemm_broadcast(s1, &r1, s2, &r2);
    if (rc == PIMHIP_ERR_UNSUPPORTED) throw NNRuntimeException(std::string("gemmBroadcast: ") + pimhip_last_error());
    check(rc);
    int t = 0;
    check(pimhip_get_gemm_type(s1, s2, &t));
    // GEMM_TYPE and PimHipGemmType hold the same integers (utils.h:30-36)
    return static_cast<GEMM_TYPE>(t);
}

struct PlanHolder {
    PimHipLstmPlan* plan = nullptr;
    int64_t max_seq_len = 0;
    int64_t hidden = 0, input_size = 0;
    std::vector<at::Tensor> params;     // what the plan reads: contiguous, kept alive
    std::vector<at::Tensor> originals;  // the caller's tensors: their addresses cannot be reused while the entry lives
    std::vector<uint32_t> versions;     // their version counters when the plan was made
    std::vector<const void*> impls;     // the caller's tensor objects (c10::TensorImpl), for the hit path below
    int64_t flags = 0;                  // has_biases | bidirectional << 1 | num_layers << 2
    uint64_t last_use = 0;
    ~PlanHolder()
    {
        if (plan) pimhip_lstm_plan_destroy(plan);
    }
};

// Plans found again by their weights.  A plan holds values derived from the weights (b_ih + b_hh, w_ih in matrix-core
// order, contiguous copies): an in-place update of a weight (seen through its version counter) makes the entry stale
// and the next call builds a new plan; updates torch does not count need pimhipInvalidateLstmPlans.  At most
// kMaxCachedPlans entries; the least recently used one goes first.
constexpr size_t kMaxCachedPlans = 64;
std::mutex g_plan_mutex;
std::map<std::vector<const void*>, std::shared_ptr<PlanHolder>> g_plans;
uint64_t g_plan_clock = 0;
// The plan of this thread's previous call.  A decoding loop calls with the same parameter list every step (the layer's
// own vector of tensors, aten_ops_executor.cpp:2218-2219): the same tensor objects, unchanged, are recognised by
// comparing pointers and version counters, without building a key, taking the lock or searching the map.
thread_local std::shared_ptr<PlanHolder> t_last_plan;
thread_local uint64_t t_last_plan_epoch = 0;
std::atomic<uint64_t> g_plan_epoch{1};  // moves whenever plans are dropped

bool sameParameterObjects(const PlanHolder& h, at::TensorList params, int64_t flags, int64_t seq_len)
{
    if (h.flags != flags || h.max_seq_len < seq_len || h.impls.size() != params.size()) return false;
    for (size_t i = 0; i < params.size(); ++i)
        if (params[i].unsafeGetTensorImpl() != h.impls[i] || params[i]._version() != h.versions[i]) return false;
    return true;
}

std::shared_ptr<PlanHolder> planFor(at::TensorList params, bool has_biases, int64_t num_layers, bool bidirectional,
                                    int64_t seq_len)
{
    const int64_t flags = (has_biases ? 1 : 0) | (bidirectional ? 2 : 0) | (num_layers << 2);
    if (t_last_plan && t_last_plan_epoch == g_plan_epoch.load(std::memory_order_acquire) &&
        sameParameterObjects(*t_last_plan, params, flags, seq_len))
        return t_last_plan;
    std::vector<const void*> key;
    for (const at::Tensor& p : params) key.push_back(p.data_ptr());
    key.push_back(reinterpret_cast<const void*>((uintptr_t)flags));
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    auto remember = [&](const std::shared_ptr<PlanHolder>& h) {
        t_last_plan = h;
        t_last_plan_epoch = g_plan_epoch.load(std::memory_order_acquire);
        return h;
    };
    auto it = g_plans.find(key);
    if (it != g_plans.end()) {
        bool fresh = it->second->versions.size() == params.size();
        for (size_t i = 0; fresh && i < params.size(); ++i) fresh = it->second->versions[i] == params[i]._version();
        if (!fresh) {
            g_plans.erase(it);
            g_plan_epoch.fetch_add(1, std::memory_order_acq_rel);
            it = g_plans.end();
        }
    }
    if (it != g_plans.end() && it->second->max_seq_len >= seq_len) {
        it->second->last_use = ++g_plan_clock;
        return remember(it->second);
    }
    auto holder = std::make_shared<PlanHolder>();
    std::vector<const void*> ptrs;
    for (const at::Tensor& p : params) {
        requireHalfOnGpu(p, "LSTM parameter");
        holder->originals.push_back(p);
        holder->versions.push_back(p._version());
        holder->impls.push_back(p.unsafeGetTensorImpl());
        holder->params.push_back(p.contiguous());
        ptrs.push_back(holder->params.back().data_ptr());
    }
    holder->flags = flags;
    const int per_cell = has_biases ? 4 : 2;
    const int64_t cells = num_layers * (bidirectional ? 2 : 1);
    if ((int64_t)params.size() != cells * per_cell) throw NNRuntimeException("unexpected number of LSTM parameter tensors");
    holder->hidden = holder->params[1].size(1);
    holder->input_size = holder->params[0].size(1);
    int64_t cap = seq_len > 16 ? seq_len : 16;
    if (it != g_plans.end() && 2 * it->second->max_seq_len > cap) cap = 2 * it->second->max_seq_len;
    check(pimhip_lstm_plan_create(&holder->plan, ptrs.data(), (int)ptrs.size(), has_biases ? 1 : 0, (int)num_layers,
                                  bidirectional ? 1 : 0, holder->input_size, holder->hidden, cap, streamOrCurrent(nullptr)));
    holder->max_seq_len = cap;
    holder->last_use = ++g_plan_clock;
    if (it != g_plans.end()) g_plan_epoch.fetch_add(1, std::memory_order_acq_rel);  // the smaller plan is replaced
    g_plans[key] = holder;
    while (g_plans.size() > kMaxCachedPlans) {
        auto oldest = g_plans.begin();
        for (auto jt = g_plans.begin(); jt != g_plans.end(); ++jt)
            if (jt->second->last_use < oldest->second->last_use) oldest = jt;
        g_plans.erase(oldest);  // a forward still holding the shared_ptr keeps its plan until it returns
        g_plan_epoch.fetch_add(1, std::memory_order_acq_rel);
    }
    return remember(holder);
}

// input holds T x input_size elements (any shape; batch 1).  y / hn / cn: defined tensors are written in place (they must be
// contiguous fp16 GPU tensors of the right number of elements), undefined ones are allocated in y_shape / state shape.
void lstmForwardInto(const at::Tensor& input, int64_t T, at::TensorList hx, at::TensorList params, bool has_biases,
                     int64_t num_layers, bool bidirectional, at::IntArrayRef y_shape, at::Tensor& y, at::Tensor& hn, at::Tensor& cn)
{
    if (hx.size() != 2) throw NNRuntimeException("hx must hold (h0, c0)");
    requireHalfOnGpu(input, "LSTM input");
    requireHalfOnGpu(hx[0], "h0");
    requireHalfOnGpu(hx[1], "c0");
    auto holder = planFor(params, has_biases, num_layers, bidirectional, T);
    const int64_t D = bidirectional ? 2 : 1;
    const int64_t H = holder->hidden;
    if (input.numel() != T * holder->input_size) throw NNRuntimeException("LSTM input width does not match w_ih");
    if (hx[0].numel() != num_layers * D * H || hx[1].numel() != num_layers * D * H)
        throw NNRuntimeException("h0 / c0 must have num_layers * num_directions * hidden_size elements");
    at::Tensor hold_x, hold_h, hold_c;
    const void* x = denseData(input, hold_x);
    const void* h0 = denseData(hx[0], hold_h);
    const void* c0 = denseData(hx[1], hold_c);
    auto dest = [&](at::Tensor& t, at::IntArrayRef shape, int64_t numel, const char* what) {
        if (!t.defined()) {
            t = at::empty(shape, input.options());
            return;
        }
        requireHalfOnGpu(t, what);
        if (!t.is_contiguous() || t.numel() != numel) throw NNRuntimeException(std::string(what) + " must be contiguous and of the result's size");
    };
    const int64_t state_shape[3] = {num_layers * D, 1, H};
    dest(y, y_shape, T * D * H, "the output buffer");
    dest(hn, state_shape, num_layers * D * H, "the hy buffer");
    dest(cn, state_shape, num_layers * D * H, "the cy buffer");
    check(pimhip_lstm_forward(holder->plan, T > 0 ? x : nullptr, h0, c0, T > 0 ? y.data_ptr() : nullptr, hn.data_ptr(),
                              cn.data_ptr(), T, streamOrCurrent(nullptr)));
}
}  // namespace

void pimhipRuntimeInitialize(int device) { check(pimhip_initialize(device)); }

int64_t pimhipInvalidateLstmPlans(at::TensorList params)
{
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    g_plan_epoch.fetch_add(1, std::memory_order_acq_rel);
    t_last_plan.reset();
    if (params.empty()) {
        const int64_t n = (int64_t)g_plans.size();
        g_plans.clear();
        return n;
    }
    int64_t n = 0;
    for (auto it = g_plans.begin(); it != g_plans.end();) {
        bool hit = false;
        for (const at::Tensor& o : it->second->originals)
            for (const at::Tensor& p : params) hit = hit || o.data_ptr() == p.data_ptr();
        if (hit) {
            it = g_plans.erase(it);
            ++n;
        } else {
            ++it;
        }
    }
    return n;
}

void pimhipRuntimeDeinitialize()
{
    {
        std::lock_guard<std::mutex> lock(g_plan_mutex);
        g_plans.clear();
        g_plan_epoch.fetch_add(1, std::memory_order_acq_rel);
        t_last_plan.reset();
    }
    check(pimhip_deinitialize());
}

static_assert((int)GEMM_TYPE::UNKNOW == PIMHIP_GEMM_UNKNOWN && (int)GEMM_TYPE::VV == PIMHIP_GEMM_VV && (int)GEMM_TYPE::MV == PIMHIP_GEMM_MV &&
                  (int)GEMM_TYPE::VM == PIMHIP_GEMM_VM && (int)GEMM_TYPE::MM == PIMHIP_GEMM_MM,
              "GEMM_TYPE and PimHipGemmType must hold the same integers");

void customAtenAddmm(std::string act_type, at::Tensor& self_tensor, at::Tensor& mat1_tensor, at::Tensor& mat2_tensor,
                     at::Scalar beta, at::Scalar alpha, torch::jit::IValue& output_iv, void* stream)
{
    requireHalfOnGpu(self_tensor, "self");
    requireHalfOnGpu(mat1_tensor, "mat1");
    requireHalfOnGpu(mat2_tensor, "mat2");
    const int dim_i0 = mat1_tensor.dim();
    const int dim_i1 = mat2_tensor.dim();
    const int dim_self = self_tensor.dim();
    const GEMM_TYPE gemm_type = classify(mat1_tensor, mat2_tensor);
    // Only "aten::relu" selects an activation (aten_ops.cpp:622-624).
    const int act = act_type == "aten::relu" ? PIMHIP_ACT_RELU : PIMHIP_ACT_NONE;

    if (gemm_type == GEMM_TYPE::VM && dim_i0 > 1) {
        // aten_ops.cpp:626-661; the IR's alpha / beta are not used on this branch (aten_ops.cpp:627-628).
        const int64_t out_w = mat2_tensor.size(dim_i1 - 1);
        const int64_t in_w = mat2_tensor.size(dim_i1 - 2);
        at::DimVector output_shape(mat1_tensor.sizes());
        output_shape[dim_i0 - 1] = out_w;
        output_shape[dim_i0 - 2] = 1;
        at::Tensor y = at::empty(output_shape, mat2_tensor.options());
        if (y.numel() != out_w) throw NNRuntimeException("VM operands do not form a single row");
        gemvInto(y, mat1_tensor, mat2_tensor, self_tensor, in_w, out_w, PIMHIP_I_X_W, act, stream);
        output_iv = torch::jit::IValue(std::move(y));
    } else if (gemm_type == GEMM_TYPE::MV && dim_i1 > 1) {
        // aten_ops.cpp:662-694
        const int64_t out_w = mat1_tensor.size(dim_i0 - 2);
        const int64_t in_w = mat1_tensor.size(dim_i0 - 1);
        at::DimVector output_shape(mat2_tensor.sizes());
        output_shape[dim_i1 - 1] = 1;
        output_shape[dim_i1 - 2] = out_w;
        at::Tensor y = at::empty(output_shape, mat1_tensor.options());
        if (y.numel() != out_w) throw NNRuntimeException("MV operands do not form a single column");
        gemvInto(y, mat2_tensor, mat1_tensor, self_tensor, in_w, out_w, PIMHIP_W_X_I, act, stream);
        output_iv = torch::jit::IValue(std::move(y));
    } else if (dim_self == 1) {
        // aten_ops.cpp:695-711: a true matrix product, LibTorch passthrough.
        at::Tensor bias = self_tensor.unsqueeze(1).repeat({1, mat2_tensor.size(dim_i1 - 1)});
        at::Tensor m2 = dim_i1 != 2 ? mat2_tensor.squeeze(0) : mat2_tensor;
        at::Tensor output = at::addmm(bias, mat1_tensor, m2, beta, alpha);
        if (act == PIMHIP_ACT_RELU) output = at::relu(output);
        for (int i = 0; i < dim_i1 - 2; ++i) output = output.unsqueeze(0);
        output_iv = torch::jit::IValue(output);
    } else {
        // aten_ops.cpp:712-757.  The reference's ENABLE_PIM branch never stores its result; the LibTorch branch is the
        // defined behaviour and is the one taken here.
        at::Tensor output = at::addmm(self_tensor, mat1_tensor, mat2_tensor, beta, alpha);
        if (act == PIMHIP_ACT_RELU) output = at::relu(output);
        output_iv = torch::jit::IValue(output);
    }
}

void customAtenMatmul(at::Tensor& self_tensor, at::Tensor& other_tensor, torch::jit::IValue& output_iv, void* stream)
{
    requireHalfOnGpu(self_tensor, "self");
    requireHalfOnGpu(other_tensor, "other");
    const int dim_i0 = self_tensor.dim();
    const int dim_i1 = other_tensor.dim();
    const GEMM_TYPE gemm_type = classify(self_tensor, other_tensor);

    if (gemm_type == GEMM_TYPE::VM) {
        // aten_ops.cpp:770-804
        const int64_t out_w = other_tensor.size(dim_i1 - 1);
        const int64_t in_w = other_tensor.size(dim_i1 - 2);
        at::DimVector output_shape(self_tensor.sizes());
        if (dim_i1 > dim_i0) {
            output_shape = at::DimVector(other_tensor.sizes());
            output_shape[dim_i1 - 1] = out_w;
            output_shape[dim_i1 - 2] = 1;
        } else {
            output_shape[dim_i0 - 1] = out_w;
            output_shape[dim_i0 - 2] = 1;
        }
        at::Tensor y = at::empty(output_shape, other_tensor.options());
        if (y.numel() != out_w) throw NNRuntimeException("VM operands do not form a single row");
        gemvInto(y, self_tensor, other_tensor, at::Tensor(), in_w, out_w, PIMHIP_I_X_W, PIMHIP_ACT_NONE, stream);
        output_iv = torch::jit::IValue(std::move(y));
    } else if (gemm_type == GEMM_TYPE::MV) {
        // aten_ops.cpp:805-840
        const int64_t out_w = self_tensor.size(dim_i0 - 2);
        const int64_t in_w = self_tensor.size(dim_i0 - 1);
        at::DimVector output_shape(other_tensor.sizes());
        if (dim_i0 > dim_i1) {
            output_shape = at::DimVector(self_tensor.sizes());
            output_shape[dim_i0 - 2] = out_w;
            output_shape.pop_back();
        } else {
            output_shape[dim_i1 - 1] = 1;
            output_shape[dim_i1 - 2] = out_w;
        }
        at::Tensor y = at::empty(output_shape, self_tensor.options());
        if (y.numel() != out_w) throw NNRuntimeException("MV operands do not form a single column");
        gemvInto(y, other_tensor, self_tensor, at::Tensor(), in_w, out_w, PIMHIP_W_X_I, PIMHIP_ACT_NONE, stream);
        output_iv = torch::jit::IValue(std::move(y));
    } else if (gemm_type == GEMM_TYPE::VV) {
        // aten_ops.cpp:841-882
        at::Tensor a = self_tensor.contiguous(), b = other_tensor.contiguous();
        int64_t in_w = 0;
        for (int i = 0; i < dim_i0; ++i) {
            if (a.size(i) != 1) {
                in_w = a.size(i);
                break;
            }
        }
        at::DimVector output_shape(other_tensor.sizes());
        if (dim_i0 > dim_i1) {
            output_shape = at::DimVector(self_tensor.sizes());
            output_shape[dim_i0 - 1] = 1;
            output_shape[dim_i0 - 2] = 1;
        } else {
            output_shape[dim_i1 - 1] = 1;
            output_shape[dim_i1 - 2] = 1;
        }
        at::Tensor output = at::empty(output_shape, a.options());
        if (output.numel() != 1 || a.numel() < in_w || b.numel() < in_w)
            throw NNRuntimeException("VV operands do not form a single dot product");
        check(pimhip_execute_dot(output.data_ptr(), a.data_ptr(), b.data_ptr(), in_w, streamOrCurrent(stream)));
        output_iv = torch::jit::IValue(output);
    } else {
        // aten_ops.cpp:883-931: LibTorch passthrough.
        output_iv = torch::jit::IValue(at::matmul(self_tensor, other_tensor));
    }
}

at::Tensor atenLinear(const at::Tensor& input, const at::Tensor& weight, const c10::optional<at::Tensor>& bias_opt)
{
    // aten_ops.cpp:304-307 (declared with the optional bias at aten_ops.h:231).  One input row: the MV product on W's
    // own row-major bytes, on torch's current stream; anything else is LibTorch's.
    if (weight.dim() != 2 || input.dim() < 1 || input.numel() != weight.size(1)) return at::linear(input, weight, bias_opt);
    const at::Tensor bias = bias_opt.has_value() ? *bias_opt : at::Tensor();
    requireHalfOnGpu(input, "input");
    requireHalfOnGpu(weight, "weight");
    requireHalfOnGpu(bias, "bias");
    at::DimVector shape(input.sizes());
    shape.back() = weight.size(0);
    at::Tensor y = at::empty(shape, weight.options());
    gemvInto(y, input, weight, bias, weight.size(1), weight.size(0), PIMHIP_W_X_I, PIMHIP_ACT_NONE, nullptr);
    return y;
}

namespace
{
int64_t lstm1SeqLen(const at::Tensor& input, bool train, bool batch_first)
{
    if (train) throw NNRuntimeException("training mode is not part of this inference path");
    if (input.dim() != 3) throw NNRuntimeException("input must be [T, 1, I] or, with batch_first, [1, T, I]");
    const int64_t batch = batch_first ? input.size(0) : input.size(1);
    if (batch != 1) throw NNRuntimeException("only batch 1 is supported (as in miopen_ops_executor.cpp:117)");
    return batch_first ? input.size(1) : input.size(0);
}
}  // namespace

std::tuple<at::Tensor, at::Tensor, at::Tensor> atenLstm1(const at::Tensor& input, at::TensorList hx,
                                                         at::TensorList params, bool has_biases, int64_t num_layers,
                                                         double /*dropout: forced to 0 by the reference, aten_ops.cpp:333*/,
                                                         bool train, bool bidirectional, bool batch_first)
{
    const int64_t T = lstm1SeqLen(input, train, batch_first);
    if (params.size() < 2) throw NNRuntimeException("unexpected number of LSTM parameter tensors");
    const int64_t DH = (bidirectional ? 2 : 1) * params[1].size(1);
    // (batch 1: [T, 1, I] and [1, T, I] are the same bytes when dense; a strided view is copied by lstmForwardInto)
    const int64_t y_shape[3] = {batch_first ? 1 : T, batch_first ? T : 1, DH};
    at::Tensor y, hn, cn;
    lstmForwardInto(input, T, hx, params, has_biases, num_layers, bidirectional, y_shape, y, hn, cn);
    return std::make_tuple(std::move(y), std::move(hn), std::move(cn));
}

void atenLstm1Into(const at::Tensor& input, at::TensorList hx, at::TensorList params, bool has_biases, int64_t num_layers,
                   double /*dropout*/, bool train, bool bidirectional, bool batch_first, at::Tensor& output, at::Tensor& hy,
                   at::Tensor& cy)
{
    const int64_t T = lstm1SeqLen(input, train, batch_first);
    if (params.size() < 2) throw NNRuntimeException("unexpected number of LSTM parameter tensors");
    const int64_t DH = (bidirectional ? 2 : 1) * params[1].size(1);
    const int64_t y_shape[3] = {batch_first ? 1 : T, batch_first ? T : 1, DH};
    lstmForwardInto(input, T, hx, params, has_biases, num_layers, bidirectional, y_shape, output, hy, cy);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> atenLstm2(const at::Tensor& data, const at::Tensor& batch_sizes,
                                                         at::TensorList hx, at::TensorList params, bool has_biases,
                                                         int64_t num_layers, double /*dropout*/, bool train,
                                                         bool bidirectional)
{
    if (train) throw NNRuntimeException("training mode is not part of this inference path");
    if (data.dim() != 2) throw NNRuntimeException("packed data must be [sum(batch_sizes), I]");
    at::Tensor bs = batch_sizes.cpu();
    if (bs.numel() != data.size(0) || !bs.eq(1).all().item<bool>())
        throw NNRuntimeException("only batch 1 packed sequences (batch_sizes all ones) are supported");
    if (params.size() < 2) throw NNRuntimeException("unexpected number of LSTM parameter tensors");
    const int64_t y_shape[2] = {data.size(0), (bidirectional ? 2 : 1) * params[1].size(1)};
    at::Tensor y, hn, cn;
    lstmForwardInto(data, data.size(0), hx, params, has_biases, num_layers, bidirectional, y_shape, y, hn, cn);
    return std::make_tuple(std::move(y), std::move(hn), std::move(cn));
}

}  // namespace op_executor
}  // namespace runtime
}  // namespace nn_compiler
