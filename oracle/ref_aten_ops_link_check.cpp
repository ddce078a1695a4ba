// Link check of the C++ operator layer against the reference's own declarations (test infrastructure).
//
// This file includes the reference's header runtime/include/executor/op_executor/aten_ops.h where it lies (it needs
// only LibTorch) and nothing of this repository.  It takes the address of every hot-path operator through that
// header's declarations, so the symbols it asks the linker for are the ones the reference's callers
// (executeAtenAddmm, executeAtenLinear, executeAtenLSTM1/2, ...) would ask for.  Linked with
// pimaicompiler_amd/cpp/aten_ops_pimhip.cpp, a definition whose signature has drifted from the reference's
// declaration is an undefined symbol and the link fails.  With -DLINK_CHECK_DRIFT the file also asks for a
// signature the reference does not declare (a control: that link has to fail).
#include <cstdio>

#include "runtime/include/executor/op_executor/aten_ops.h"

namespace ops = nn_compiler::runtime::op_executor;

#ifdef LINK_CHECK_DRIFT
namespace nn_compiler { namespace runtime { namespace op_executor {
at::Tensor atenLinear(const at::Tensor& input, const at::Tensor& weight, const at::Tensor& bias);
}}}
#endif

int main()
{
    // aten_ops.h:231, 241-249, 434-437
    at::Tensor (*linear)(const at::Tensor&, const at::Tensor&, const c10::optional<at::Tensor>&) = &ops::atenLinear;
    auto* lstm1 = &ops::atenLstm1;
    auto* lstm2 = &ops::atenLstm2;
    auto* addmm = &ops::customAtenAddmm;
    auto* matmul = &ops::customAtenMatmul;
    const void* table[] = {(const void*)linear, (const void*)lstm1, (const void*)lstm2, (const void*)addmm, (const void*)matmul,
#ifdef LINK_CHECK_DRIFT
                           (const void*)static_cast<at::Tensor (*)(const at::Tensor&, const at::Tensor&, const at::Tensor&)>(&ops::atenLinear),
#endif
    };
    int n = 0;
    for (const void* p : table) n += p != nullptr;
    std::printf("%d hot-path operators resolved through the reference's aten_ops.h\n", n);
    return n == (int)(sizeof(table) / sizeof(table[0])) ? 0 : 1;
}
