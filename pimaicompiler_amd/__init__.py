"""MI355X (gfx950) implementation of the PimAiCompiler runtime's memory-bound hot path.

The compute lives in libpimhip.so (hand-written HIP kernels behind the C ABI of include/pimhip.h).
`pimaicompiler_amd.ops` mirrors the reference runtime's operator interface for this path on torch tensors,
which are used for device memory and streams only.
"""
from . import _lib  # noqa: F401
from . import executor, io, rewrite  # noqa: F401
from .ops import (  # noqa: F401
    NNRuntimeException,
    GemmType,
    initialize,
    deinitialize,
    gemm_broadcast,
    get_gemm_type,
    custom_aten_addmm,
    custom_aten_matmul,
    aten_linear,
    aten_linear_cat2,
    aten_bmm,
    aten_add,
    aten_lstm1,
    aten_lstm2,
    execute_gemv_group,
    input_projection,
    input_projection_packed,
    pack_projection_weight,
    LstmPlan,
    DecoderPlan,
    MoePlan,
    RnntPlan,
    prepare_lstm,
    invalidate_lstm_plans,
    gemv_status,
    gemv_fallbacks,
    synchronize_and_check,
    set_gemv_spin_limit,
)
