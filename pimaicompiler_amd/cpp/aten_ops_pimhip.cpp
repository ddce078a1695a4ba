// Bodies for the reference's GEMV / LSTM operators on top of libpimhip.so (see aten_ops_pimhip.h).
// Dispatch rules and output shapes follow runtime/source/executor/op_executor/aten_ops.cpp:609-932; the arithmetic is in
// the HIP kernels behind the C ABI.  at::Tensor is used for device memory only.
#include "aten_ops_pimhip.h"

#include <c10/hip/HIPStream.h>

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

// A 2-D weight usable without a copy.  `flipped` is set when the view is the transpose of a row-major matrix, i.e.
// the other operand order on the same bytes (what SwapAddmmInputs hands over); anything else is made contiguous.
at::Tensor weightView(const at::Tensor& w, bool& flipped)
{
    flipped = false;
    if (w.is_contiguous()) return w;
    if (w.dim() == 2 && w.stride(0) == 1 && w.stride(1) >= w.size(0)) {
        flipped = true;
        return w.t();
    }
    return w.contiguous();
}

at::Tensor gemv(const at::Tensor& x, const at::Tensor& weight2d, const at::Tensor& bias, int64_t in_w, int64_t out_w,
                int order, int act, void* stream)
{
    bool flipped = false;
    at::Tensor w = weightView(weight2d, flipped);
    if (flipped) order = (order == PIMHIP_I_X_W) ? PIMHIP_W_X_I : PIMHIP_I_X_W;
    const int64_t ld = w.size(0) > 1 ? w.stride(0) : w.size(1);
    at::Tensor xc = x.contiguous();
    at::Tensor bc = bias.defined() ? bias.contiguous() : bias;
    if (bc.defined() && bc.numel() != out_w) throw NNRuntimeException("bias length does not match the GEMV output");
    at::Tensor out = at::empty({out_w}, w.options());
    check(pimhip_execute_gemv(out.data_ptr(), xc.data_ptr(), w.data_ptr(), bc.defined() ? bc.data_ptr() : nullptr, in_w,
                              out_w, ld, act, order, streamOrCurrent(stream)));
    return out;
}

struct PlanHolder {
    PimHipLstmPlan* plan = nullptr;
    int64_t max_seq_len = 0;
    std::vector<at::Tensor> params;     // what the plan reads: contiguous, kept alive
    std::vector<at::Tensor> originals;  // the caller's tensors: their addresses cannot be reused while the entry lives
    std::vector<uint32_t> versions;     // their version counters when the plan was made
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

std::shared_ptr<PlanHolder> planFor(at::TensorList params, bool has_biases, int64_t num_layers, bool bidirectional,
                                    int64_t seq_len)
{
    std::vector<const void*> key;
    for (const at::Tensor& p : params) key.push_back(p.data_ptr());
    key.push_back(reinterpret_cast<const void*>((uintptr_t)((has_biases ? 1 : 0) | (bidirectional ? 2 : 0) | (num_layers << 2))));
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) {
        bool fresh = it->second->versions.size() == params.size();
        for (size_t i = 0; fresh && i < params.size(); ++i) fresh = it->second->versions[i] == params[i]._version();
        if (!fresh) {
            g_plans.erase(it);
            it = g_plans.end();
        }
    }
    if (it != g_plans.end() && it->second->max_seq_len >= seq_len) {
        it->second->last_use = ++g_plan_clock;
        return it->second;
    }
    auto holder = std::make_shared<PlanHolder>();
    std::vector<const void*> ptrs;
    for (const at::Tensor& p : params) {
        requireHalfOnGpu(p, "LSTM parameter");
        holder->originals.push_back(p);
        holder->versions.push_back(p._version());
        holder->params.push_back(p.contiguous());
        ptrs.push_back(holder->params.back().data_ptr());
    }
    const int per_cell = has_biases ? 4 : 2;
    const int64_t cells = num_layers * (bidirectional ? 2 : 1);
    if ((int64_t)params.size() != cells * per_cell) throw NNRuntimeException("unexpected number of LSTM parameter tensors");
    const int64_t hidden = holder->params[1].size(1);
    const int64_t input_size = holder->params[0].size(1);
    int64_t cap = seq_len > 16 ? seq_len : 16;
    if (it != g_plans.end() && 2 * it->second->max_seq_len > cap) cap = 2 * it->second->max_seq_len;
    check(pimhip_lstm_plan_create(&holder->plan, ptrs.data(), (int)ptrs.size(), has_biases ? 1 : 0, (int)num_layers,
                                  bidirectional ? 1 : 0, input_size, hidden, cap, streamOrCurrent(nullptr)));
    holder->max_seq_len = cap;
    holder->last_use = ++g_plan_clock;
    g_plans[key] = holder;
    while (g_plans.size() > kMaxCachedPlans) {
        auto oldest = g_plans.begin();
        for (auto jt = g_plans.begin(); jt != g_plans.end(); ++jt)
            if (jt->second->last_use < oldest->second->last_use) oldest = jt;
        g_plans.erase(oldest);  // a forward still holding the shared_ptr keeps its plan until it returns
    }
    return holder;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> lstmForward(const at::Tensor& x2d, at::TensorList hx, at::TensorList params,
                                                           bool has_biases, int64_t num_layers, bool bidirectional)
{
    if (hx.size() != 2) throw NNRuntimeException("hx must hold (h0, c0)");
    requireHalfOnGpu(x2d, "LSTM input");
    requireHalfOnGpu(hx[0], "h0");
    requireHalfOnGpu(hx[1], "c0");
    const int64_t T = x2d.size(0);
    auto holder = planFor(params, has_biases, num_layers, bidirectional, T);
    const int64_t D = bidirectional ? 2 : 1;
    const int64_t H = holder->params[1].size(1);
    if (x2d.size(1) != holder->params[0].size(1)) throw NNRuntimeException("LSTM input width does not match w_ih");
    if (hx[0].numel() != num_layers * D * H || hx[1].numel() != num_layers * D * H)
        throw NNRuntimeException("h0 / c0 must have num_layers * num_directions * hidden_size elements");
    at::Tensor x = x2d.contiguous(), h0 = hx[0].contiguous(), c0 = hx[1].contiguous();
    at::Tensor y = at::empty({T, D * H}, x.options());
    at::Tensor hn = at::empty({num_layers * D, 1, H}, x.options());
    at::Tensor cn = at::empty({num_layers * D, 1, H}, x.options());
    check(pimhip_lstm_forward(holder->plan, T > 0 ? x.data_ptr() : nullptr, h0.data_ptr(), c0.data_ptr(),
                              T > 0 ? y.data_ptr() : nullptr, hn.data_ptr(), cn.data_ptr(), T, streamOrCurrent(nullptr)));
    return std::make_tuple(y, hn, cn);
}
}  // namespace

void pimhipRuntimeInitialize(int device) { check(pimhip_initialize(device)); }

int64_t pimhipInvalidateLstmPlans(at::TensorList params)
{
    std::lock_guard<std::mutex> lock(g_plan_mutex);
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
    }
    check(pimhip_deinitialize());
}

void customAtenAddmm(std::string act_type, at::Tensor& self_tensor, at::Tensor& mat1_tensor, at::Tensor& mat2_tensor,
                     at::Scalar beta, at::Scalar alpha, torch::jit::IValue& output_iv, void* stream)
{
    requireHalfOnGpu(self_tensor, "self");
    requireHalfOnGpu(mat1_tensor, "mat1");
    requireHalfOnGpu(mat2_tensor, "mat2");
    const int dim_i0 = mat1_tensor.dim();
    const int dim_i1 = mat2_tensor.dim();
    const int dim_self = self_tensor.dim();
    auto mat1_shape = mat1_tensor.sizes().vec();
    auto mat2_shape = mat2_tensor.sizes().vec();
    utils::gemmBroadcast(mat1_shape, mat2_shape);
    const GEMM_TYPE gemm_type = utils::getGemmType(mat1_shape, mat2_shape);
    // Only "aten::relu" selects an activation (aten_ops.cpp:622-624).
    const int act = act_type == "aten::relu" ? PIMHIP_ACT_RELU : PIMHIP_ACT_NONE;

    if (gemm_type == GEMM_TYPE::VM && dim_i0 > 1) {
        // aten_ops.cpp:626-661; the IR's alpha / beta are not used on this branch (aten_ops.cpp:627-628).
        const int64_t out_w = mat2_tensor.size(dim_i1 - 1);
        const int64_t in_w = mat2_tensor.size(dim_i1 - 2);
        at::Tensor y = gemv(mat1_tensor.reshape({-1}), mat2_tensor.reshape({in_w, out_w}), self_tensor.reshape({-1}), in_w,
                            out_w, PIMHIP_I_X_W, act, stream);
        auto output_shape = mat1_tensor.sizes().vec();
        output_shape[dim_i0 - 1] = out_w;
        output_shape[dim_i0 - 2] = 1;
        output_iv = torch::jit::IValue(y.view(output_shape));
    } else if (gemm_type == GEMM_TYPE::MV && dim_i1 > 1) {
        // aten_ops.cpp:662-694
        const int64_t out_w = mat1_tensor.size(dim_i0 - 2);
        const int64_t in_w = mat1_tensor.size(dim_i0 - 1);
        at::Tensor y = gemv(mat2_tensor.reshape({-1}), mat1_tensor.reshape({out_w, in_w}), self_tensor.reshape({-1}), in_w,
                            out_w, PIMHIP_W_X_I, act, stream);
        auto output_shape = mat2_tensor.sizes().vec();
        output_shape[dim_i1 - 1] = 1;
        output_shape[dim_i1 - 2] = out_w;
        output_iv = torch::jit::IValue(y.view(output_shape));
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
    auto self_shape = self_tensor.sizes().vec();
    auto other_shape = other_tensor.sizes().vec();
    utils::gemmBroadcast(self_shape, other_shape);
    const GEMM_TYPE gemm_type = utils::getGemmType(self_shape, other_shape);

    if (gemm_type == GEMM_TYPE::VM) {
        // aten_ops.cpp:770-804
        const int64_t out_w = other_tensor.size(dim_i1 - 1);
        const int64_t in_w = other_tensor.size(dim_i1 - 2);
        at::Tensor y = gemv(self_tensor.reshape({-1}), other_tensor.reshape({in_w, out_w}), at::Tensor(), in_w, out_w,
                            PIMHIP_I_X_W, PIMHIP_ACT_NONE, stream);
        auto output_shape = self_tensor.sizes().vec();
        if (dim_i1 > dim_i0) {
            output_shape = other_tensor.sizes().vec();
            output_shape[dim_i1 - 1] = out_w;
            output_shape[dim_i1 - 2] = 1;
        } else {
            output_shape[dim_i0 - 1] = out_w;
            output_shape[dim_i0 - 2] = 1;
        }
        output_iv = torch::jit::IValue(y.view(output_shape));
    } else if (gemm_type == GEMM_TYPE::MV) {
        // aten_ops.cpp:805-840
        const int64_t out_w = self_tensor.size(dim_i0 - 2);
        const int64_t in_w = self_tensor.size(dim_i0 - 1);
        at::Tensor y = gemv(other_tensor.reshape({-1}), self_tensor.reshape({out_w, in_w}), at::Tensor(), in_w, out_w,
                            PIMHIP_W_X_I, PIMHIP_ACT_NONE, stream);
        auto output_shape = other_tensor.sizes().vec();
        if (dim_i0 > dim_i1) {
            output_shape = self_tensor.sizes().vec();
            output_shape[dim_i0 - 2] = out_w;
            output_shape.pop_back();
        } else {
            output_shape[dim_i1 - 1] = 1;
            output_shape[dim_i1 - 2] = out_w;
        }
        output_iv = torch::jit::IValue(y.view(output_shape));
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
        auto output_shape = other_tensor.sizes().vec();
        if (dim_i0 > dim_i1) {
            output_shape = self_tensor.sizes().vec();
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
    if (weight.dim() != 2 || input.numel() != weight.size(1)) return at::linear(input, weight, bias_opt);
    const at::Tensor bias = bias_opt.has_value() ? *bias_opt : at::Tensor();
    requireHalfOnGpu(input, "input");
    requireHalfOnGpu(weight, "weight");
    requireHalfOnGpu(bias, "bias");
    at::Tensor y = gemv(input.reshape({-1}), weight, bias, weight.size(1), weight.size(0), PIMHIP_W_X_I, PIMHIP_ACT_NONE, nullptr);
    auto shape = input.sizes().vec();
    shape.back() = weight.size(0);
    return y.view(shape);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> atenLstm1(const at::Tensor& input, at::TensorList hx,
                                                         at::TensorList params, bool has_biases, int64_t num_layers,
                                                         double /*dropout: forced to 0 by the reference, aten_ops.cpp:333*/,
                                                         bool train, bool bidirectional, bool batch_first)
{
    if (train) throw NNRuntimeException("training mode is not part of this inference path");
    if (input.dim() != 3) throw NNRuntimeException("input must be [T, 1, I] or, with batch_first, [1, T, I]");
    const int64_t batch = batch_first ? input.size(0) : input.size(1);
    if (batch != 1) throw NNRuntimeException("only batch 1 is supported (as in miopen_ops_executor.cpp:117)");
    const int64_t T = batch_first ? input.size(1) : input.size(0);
    auto out = lstmForward(input.reshape({T, input.size(2)}), hx, params, has_biases, num_layers, bidirectional);
    at::Tensor y = std::get<0>(out);
    y = batch_first ? y.view({1, T, y.size(1)}) : y.view({T, 1, y.size(1)});
    return std::make_tuple(y, std::get<1>(out), std::get<2>(out));
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
    return lstmForward(data, hx, params, has_biases, num_layers, bidirectional);
}

}  // namespace op_executor
}  // namespace runtime
}  // namespace nn_compiler
