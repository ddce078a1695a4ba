// C++ host side of the GEMV / LSTM hot path with the reference runtime's own signatures, on top of the C ABI of
// include/pimhip.h.  A maintainer of the reference replaces the bodies of these functions in
// runtime/source/executor/op_executor/aten_ops.cpp (declarations in
// runtime/include/executor/op_executor/aten_ops.h:231-249, 434-437) and
// runtime/source/executor/utils/utils.cpp:293-396 by the ones in aten_ops_pimhip.cpp; callers
// (executeAtenAddmm, executeAtenMatmul, executeAtenLSTM1/2, ...) stay as they are.
#pragma once

#include <torch/script.h>

#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

namespace nn_compiler
{
namespace runtime
{
namespace utils
{
// runtime/include/executor/utils/utils.h:30-36: a plain enum, enumerators in this order (MV = 2, VM = 3).
enum GEMM_TYPE {
    UNKNOW,
    VV,  // Vector * Vector
    MV,  // Matrix * Vector
    VM,  // Vector * Matrix
    MM   // Matrix * Matrix
};

// runtime/include/executor/utils/utils.h:166-176
class NNRuntimeException : public std::runtime_error
{
   public:
    explicit NNRuntimeException(const std::string& msg) : std::runtime_error(msg) {}
};

void gemmBroadcast(std::vector<int64_t>& shape1, std::vector<int64_t>& shape2);
GEMM_TYPE getGemmType(std::vector<int64_t> self_shape, std::vector<int64_t> other_shape);
}  // namespace utils

namespace op_executor
{
// One call per device before the first operator (PimInitialize in NNRuntime's constructor, nn_runtime.cpp:32) and
// once at the end (PimDeinitialize, nn_runtime.cpp:85).
void pimhipRuntimeInitialize(int device);
void pimhipRuntimeDeinitialize();

// atenLstm1/2 keep one prepared plan per set of weight tensors (the place of the packed MIOpen buffer the reference's
// ModelBuilder builds once, runtime/source/builder/model_builder.cpp:226-319).  A plan is rebuilt when torch's
// version counter of a weight has moved; weights changed behind torch's back need this call, which drops the plans
// made from any of `params` (all plans for an empty list) and returns how many it dropped.
int64_t pimhipInvalidateLstmPlans(at::TensorList params);

void customAtenAddmm(std::string act_type, at::Tensor& self_tensor, at::Tensor& mat1_tensor, at::Tensor& mat2_tensor,
                     at::Scalar beta, at::Scalar alpha, torch::jit::IValue& output_iv, void* stream = nullptr);

void customAtenMatmul(at::Tensor& self_tensor, at::Tensor& other_tensor, torch::jit::IValue& output_iv,
                      void* stream = nullptr);

at::Tensor atenLinear(const at::Tensor& input, const at::Tensor& weight, const c10::optional<at::Tensor>& bias = {});

std::tuple<at::Tensor, at::Tensor, at::Tensor> atenLstm1(const at::Tensor& input, at::TensorList hx,
                                                         at::TensorList params, bool has_biases, int64_t num_layers,
                                                         double dropout, bool train, bool bidirectional,
                                                         bool batch_first);

// atenLstm1 with results written where the caller wants them: `output`, `hy`, `cy` that are defined (contiguous fp16 GPU
// tensors with the results' element counts, e.g. rows of the decoder's state buffer or the head of an attention
// concatenation buffer) are filled in place, undefined ones are allocated.  It takes the place of the at::cat / slice /
// updateBlob sequence executeAtenLSTM1 runs after every GNMT decoder step to move hy / cy / output into those buffers
// (aten_ops_executor.cpp:2238-2302), and of the three allocations per call.  The outputs must not overlap the inputs.
void atenLstm1Into(const at::Tensor& input, at::TensorList hx, at::TensorList params, bool has_biases, int64_t num_layers,
                   double dropout, bool train, bool bidirectional, bool batch_first, at::Tensor& output, at::Tensor& hy,
                   at::Tensor& cy);

std::tuple<at::Tensor, at::Tensor, at::Tensor> atenLstm2(const at::Tensor& data, const at::Tensor& batch_sizes,
                                                         at::TensorList hx, at::TensorList params, bool has_biases,
                                                         int64_t num_layers, double dropout, bool train,
                                                         bool bidirectional);
}  // namespace op_executor
}  // namespace runtime
}  // namespace nn_compiler
