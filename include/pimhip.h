/*
 * pimhip.h -- C ABI of the MI355X (gfx950) hot path of the PimAiCompiler runtime: the fp16 batch-1
 * GEMV family and the LSTM cell stack.
 *
 * Every entry point replaces one piece of the interface the reference runtime reaches this path
 * through (paths relative to the reference tree):
 *   - the PIM SDK calls made by customAtenAddmm / customAtenMatmul
 *     (runtime/source/executor/op_executor/aten_ops.cpp:609-932), i.e. PimCreateGemmDesc /
 *     PimCreateBo / PimExecuteGemm / PimDestroy*;
 *   - the LSTM forward of executeAtenLSTM1/2 and executeMIOpenLSTM1/2
 *     (runtime/source/executor/op_executor/aten_ops_executor.cpp:2135-2399,
 *      runtime/source/executor/op_executor/miopen_ops_executor.cpp:22-421);
 *   - the shape logic gemmBroadcast / getGemmType
 *     (runtime/source/executor/utils/utils.cpp:293-396).
 *
 * Conventions
 *   - All data pointers are device pointers on the current HIP device unless a parameter says
 *     "host".  fp16 tensors are IEEE binary16, densely packed unless a leading dimension is given.
 *   - `stream` is a hipStream_t passed as void* (the reference passes streams the same way,
 *     aten_ops.h:434-437); NULL means the null stream.  Every entry point enqueues on `stream`
 *     and returns without synchronising, unless stated otherwise.
 *   - The caller owns every buffer.  Nothing here allocates the outputs.
 *   - Return value: PIMHIP_OK (0) or a PimHipStatus error; pimhip_last_error() returns a
 *     thread-local description of the last failure.  Unsupported arguments are reported, never
 *     silently ignored (the reference's launchers `return` silently, custom_ops.h:126-129).
 *   - The library keeps per-device state only (workspaces keyed by device and stream).  Calls on
 *     different streams may run concurrently; calls on one stream are ordered by that stream.
 */
#ifndef PIMHIP_H_
#define PIMHIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum PimHipStatus {
    PIMHIP_OK = 0,
    PIMHIP_ERR_INVALID_ARGUMENT = 1,
    PIMHIP_ERR_UNSUPPORTED = 2,
    PIMHIP_ERR_HIP = 3,
    PIMHIP_ERR_NOT_INITIALIZED = 4,
    PIMHIP_ERR_TIMEOUT = 5
} PimHipStatus;

/* Activation fused into the GEMV epilogue.  Mirrors PimActFunc {NONE, ACT_RELU} (aten_ops.cpp:615-624). */
typedef enum PimHipActFunc { PIMHIP_ACT_NONE = 0, PIMHIP_ACT_RELU = 1 } PimHipActFunc;

/* Operand order of a GEMV.  Mirrors the PIM SDK's I_X_W / W_X_I (aten_ops.cpp:653,686). */
typedef enum PimHipGemmOrder {
    PIMHIP_I_X_W = 0, /* y[1,out] = x[1,in] . A[in,out]   ("VM") */
    PIMHIP_W_X_I = 1  /* y[out,1] = A[out,in] . x[in,1]   ("MV") */
} PimHipGemmOrder;

/* Shape classes of a matrix product.  Same enumerators in the same order, hence the same integers, as GEMM_TYPE
 * {UNKNOW, VV, MV, VM, MM} (runtime/include/executor/utils/utils.h:30-36). */
typedef enum PimHipGemmType {
    PIMHIP_GEMM_UNKNOWN = 0,
    PIMHIP_GEMM_VV = 1, /* vector . vector */
    PIMHIP_GEMM_MV = 2, /* matrix . vector */
    PIMHIP_GEMM_VM = 3, /* vector . matrix */
    PIMHIP_GEMM_MM = 4
} PimHipGemmType;

/* ---- init / teardown ------------------------------------------------------------------------ */

/* Replaces PimInitialize(RT_TYPE_HIP, PIM_FP16) (runtime/source/nn_runtime.cpp:32).  Binds the library
 * to `device` (a HIP ordinal), checks that it is a gfx950 part and creates its per-device state.
 * May be called once per device; repeated calls are no-ops. */
int pimhip_initialize(int device);

/* Replaces PimDeinitialize() (runtime/source/nn_runtime.cpp:85).  Synchronises every initialised device
 * and frees all workspaces and LSTM plans' internal buffers owned by the library. */
int pimhip_deinitialize(void);

/* Thread-local text of the last error returned on this thread ("" if none). */
const char* pimhip_last_error(void);

/* ---- shape logic (host, integer only) ------------------------------------------------------- */

/* Replaces gemmBroadcast (utils.cpp:293-371): pads two matmul operand shapes towards rank 4.
 * shape1/shape2 are host arrays with room for 4 entries; rank1/rank2 are in/out.  Shapes the reference
 * leaves at a rank other than 4 (it would then read out of range in getGemmType) are returned
 * as they are with PIMHIP_ERR_UNSUPPORTED; ranks above 4 or below 1 give PIMHIP_ERR_INVALID_ARGUMENT. */
int pimhip_gemm_broadcast(int64_t* shape1, int* rank1, int64_t* shape2, int* rank2);

/* Replaces getGemmType (utils.cpp:373-396) on two rank-4 shapes; writes a PimHipGemmType. */
int pimhip_get_gemm_type(const int64_t* self_shape4, const int64_t* other_shape4, int* gemm_type);

/* ---- fp16 GEMV family ----------------------------------------------------------------------- */

/* Replaces PimCreateGemmDesc + 4x PimCreateBo + PimExecuteGemm + destroys for the batch-1 cases
 * (aten_ops.cpp:647-659, 680-692, 792-802, 828-838).
 *   order == PIMHIP_W_X_I: weight is [out_w, in_w] row-major with row pitch ld_weight (elements)
 *   order == PIMHIP_I_X_W: weight is [in_w, out_w] row-major with row pitch ld_weight (elements)
 * out[out_w] = act(sum_k weight * in[k] + bias[out_w]); bias may be NULL.  fp32 accumulation, one
 * rounding to fp16 at the store.  As in the reference's VM/MV branches there is no alpha/beta
 * (aten_ops.cpp:627-628).  ld_weight == 0 selects the dense pitch.
 * The I_X_W order splits the reduction over blocks for all but small weights; the blocks exchange partial sums through
 * a per-stream workspace the library allocates on the first such call on a stream (the call synchronises that stream
 * then, and again whenever a later call needs a larger workspace).  Calls that share a stream must not overlap.  Every
 * wait inside the kernel is bounded, and one that gives up costs time, not the result: the block computes the missing
 * partial sums itself, in the order their own block would have, so the result has the bits it would have had
 * (pimhip_gemv_fallbacks counts such events; the next I_X_W call on that stream outside a graph capture puts the workspace
 * back in order, synchronising the stream once). */
int pimhip_execute_gemv(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                        int64_t out_w, int64_t ld_weight, int act, int order, void* stream);

/* The same with the alpha and beta of the reference's own HIP launchers (rocblas_gemv_template_xAy / _Axy,
 * rocblas_addmv_template_xAy / _Axy, runtime/include/executor/op_executor/custom_ops.h:123-139, 198-214, 281-298, 364-381):
 * out[out_w] = act(alpha * sum_k weight * in[k] + beta * out[out_w] + bias[out_w]); out is not read when beta == 0.
 * alpha == 1, beta == 0 (the only values the reference passes, aten_ops.cpp:627-628, custom_op_ut.cpp:26-27) is
 * pimhip_execute_gemv itself; other values take plain kernels (2-byte loads, any size, pitch and alignment) that run at a
 * fraction of its rate. */
int pimhip_execute_gemv_scaled(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                               int64_t out_w, int64_t ld_weight, int act, int order, float alpha, float beta, void* stream);

/* out[out_w] = act(weight[out_w, in1_w + in2_w] . cat(in1, in2) + bias) without the concatenation (order W_X_I): in1 and
 * in2 lie apart, as the encoder frame and the prediction that the RNNT joint network's first layer reads do.  Replaces the
 * pair of dependent products RemoveCatForAddmm makes of such a layer
 * (compiler/source/frontend/optimizer/remove_cat_for_addmm.cpp:46-191) by one launch on the whole weight.  in1_w, in2_w and
 * ld_weight (0 = dense) must be multiples of 8 and in1, in2, weight 16-byte aligned (PIMHIP_ERR_UNSUPPORTED otherwise). */
int pimhip_execute_gemv_cat2(void* out, const void* in1, int64_t in1_w, const void* in2, int64_t in2_w, const void* weight,
                             const void* bias, int64_t out_w, int64_t ld_weight, int act, void* stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  Same arguments, result and bits as pimhip_execute_gemv,
 * but the partial sums of a sliced I_X_W product go through a 256 KiB array that is part of the library's
 * image on every GPU it runs on, instead of a per-stream workspace: the call allocates, frees and synchronises
 * nothing and records kernels only.  A product that needs more than 65536 partial sums
 * ((slices - 1) * out_w; none that pimhip_execute_gemv slices on a 256-CU part does) is refused with
 * PIMHIP_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that may overlap there (different streams,
 * or replays of graphs holding such calls) race and must be ordered by the caller.  A wait that gives up is made good
 * inside the launch as in pimhip_execute_gemv; the next call outside a graph capture refills the array (the one case in
 * which this entry point synchronises the stream). */
int pimhip_execute_gemv_static(void* out, const void* in, const void* weight, const void* bias, int64_t in_w,
                               int64_t out_w, int64_t ld_weight, int act, int order, void* stream);

/* Replaces the VV branch of customAtenMatmul (aten_ops.cpp:841-882): out[0] = sum_k a[k] * b[k]. */
int pimhip_execute_dot(void* out, const void* a, const void* b, int64_t in_w, void* stream);

/* Replaces executeMultiStream's N sibling GEMVs on N streams
 * (runtime/source/executor/op_executor/stream_ops_executor.cpp:27-50) by one grouped launch on one
 * stream.  All arrays are host arrays of `count` entries (count <= 64); entries follow
 * pimhip_execute_gemv's meaning and all use order PIMHIP_W_X_I. */
int pimhip_execute_gemv_group(int count, void* const* outs, const void* const* ins, const void* const* weights,
                              const void* const* biases, const int64_t* in_ws, const int64_t* out_ws,
                              const int* acts, void* stream);

/* Replaces rocblas_bmm_template_xAy and the two device copies that follow it in executeAtenBmm
 * (runtime/include/executor/op_executor/custom_ops.h:435-466,
 *  runtime/source/executor/op_executor/aten_ops_executor.cpp:668-747): y[1, n] = x[1, k] . A[k, n], A row-major and
 * dense, fp32 accumulation (the reference accumulates in fp16), the result stored to every one of the n_outs
 * (1..4) buffers of the host array `outs` (the GNMT attention context lands in three concatenation buffers). */
int pimhip_execute_bmm(void* const* outs, int n_outs, const void* x, const void* A, int64_t k, int64_t n, void* stream);

/* Replaces custom_add (custom_ops.h:383-433; executeAtenAdd, aten_ops_executor.cpp:43-179):
 * c[m, n] = a[m, n] + b, with b [m, n] (b_broadcast == 0) or one row [n] added to every row (b_broadcast != 0).
 * fp16 in and out, each sum rounded once; c may alias a or b; any n (the reference needs n % 4 == 0). */
int pimhip_execute_add(void* c, const void* a, const void* b, int64_t m, int64_t n, int b_broadcast, void* stream);

/* ---- LSTM ----------------------------------------------------------------------------------- */

typedef struct PimHipLstmPlan PimHipLstmPlan;

/* One-time weight preparation; replaces ModelBuilder::buildLstmParameterVector / reArangeLstmWeights
 * (runtime/source/builder/model_builder.cpp:158-319) and the per-call MIOpen descriptor and workspace
 * set-up (miopen_ops_executor.cpp:109-160).
 *   params: host array of n_params device pointers in LibTorch order, per layer then per direction
 *           (w_ih [4H, I_l], w_hh [4H, H], then b_ih [4H], b_hh [4H] when has_biases), gate order
 *           (i, f, g, o); I_0 = input_size, I_l = num_directions * H for l > 0.
 * The plan keeps the caller's weight pointers (they must outlive the plan), pre-adds b_ih + b_hh, copies the w_ih of
 * the layers whose input projection runs as a batch into the matrix cores' fragment order (one more w_ih of memory
 * for those layers), and owns the internal buffers for up to max_seq_len steps.  Runs on `stream` and synchronises it. */
int pimhip_lstm_plan_create(PimHipLstmPlan** plan, const void* const* params, int n_params, int has_biases,
                            int num_layers, int bidirectional, int64_t input_size, int64_t hidden_size,
                            int64_t max_seq_len, void* stream);

int pimhip_lstm_plan_destroy(PimHipLstmPlan* plan);

/* Replaces atenLstm1 / atenLstm2 with batch 1 (aten_ops.cpp:328-344) and miopenRNNForwardInference
 * (miopen_ops_executor.cpp:175,230,393,411).  Inference only (dropout is forced to 0 by the reference,
 * aten_ops.cpp:333,342).
 *   x  [seq_len, input_size]            (batch 1: the same bytes for [T,1,I], [1,T,I] and packed [T,I])
 *   h0, c0 [num_layers*num_directions, hidden_size]
 *   y  [seq_len, num_directions*hidden_size]
 *   hn, cn [num_layers*num_directions, hidden_size], ordered (l0 fwd, l0 bwd, l1 fwd, ...)
 * y, hn, cn may not alias x, h0, c0.  Calls sharing one plan must be ordered on one stream.  Sequences of two or more
 * steps run in a kernel that needs all its blocks resident at once: a call on another stream than the device's
 * previous such call is ordered after it (an event wait), so that two of them never share the GPU.  On a capturing
 * stream that wait is left out (a graph cannot wait for another stream's event): order replays of such a graph against
 * the device's other sequence calls yourself.  The call records kernels only; the one case a graph must not hold, the
 * re-initialisation of the plan's buffers after a change of mode, returns PIMHIP_ERR_UNSUPPORTED there. */
int pimhip_lstm_forward(PimHipLstmPlan* plan, const void* x, const void* h0, const void* c0, void* y, void* hn,
                        void* cn, int64_t seq_len, void* stream);

/* After the stream has been synchronised.  PIMHIP_OK unless the workgroups of the per-XCD kernel (mode 4) were not dealt to
 * the XCDs in rotation in some forward of this plan (PIMHIP_ERR_TIMEOUT, reported once, here or by the next
 * pimhip_lstm_forward; that forward's outputs are undefined and the plan stops choosing that kernel; a probe launch at
 * plan creation keeps the kernel from being offered where the placement is not a rotation to begin with).  A wait that
 * gave up is not an error: see pimhip_lstm_plan_fallbacks. */
int pimhip_lstm_plan_status(PimHipLstmPlan* plan);

/* No counterpart in the reference.  The workgroups of the persistent sequence kernels wait for one another, every wait
 * bounded (pimhip_lstm_plan_set_spin_limit, and one second).  A wait that gives up (other work kept part of the GPU from
 * running the workgroups together) costs time, not the result: the workgroup stops publishing, and at the end of the launch
 * computes its units of the recurrence by itself from the call's inputs, so y, hn and cn are what they would have been.
 * Sequence launches after that run the same way from their start until a pimhip_lstm_forward issued outside a graph capture
 * has re-initialised the exchange (it synchronises the stream then); after the third such event the plan runs one launch
 * per step, whose workgroups wait for nobody.
 *   *events: waits that have given up so far, as far as the host has seen (ask after synchronising the stream);
 *   *exchanging (may be null): 1 while sequence calls still use the persistent kernels, 0 once they do not. */
int pimhip_lstm_plan_fallbacks(PimHipLstmPlan* plan, uint64_t* events, int* exchanging);

/* Upper bound on the polls of one wait inside the persistent kernels (default 2^22, roughly seconds).  Tests of the path
 * above pass 0 here so that every wait whose first look fails gives up at once; every kernel still ends by itself. */
int pimhip_lstm_plan_set_spin_limit(PimHipLstmPlan* plan, unsigned int spin_limit);

/* Selects how pimhip_lstm_forward runs the recurrence: 0 = automatic, 1 = one fused launch per step,
 * 2 = persistent sequence kernel (hidden_size up to 2048; fails with PIMHIP_ERR_UNSUPPORTED otherwise), 3 = as 2 but with
 * four hidden units per block in every launch (2 runs a single unidirectional layer with eight), 4 = every recurrence
 * (layer and direction) on one XCD of the part, the two directions of a layer side by side on two, the layers of a
 * unidirectional stack as a pipeline (hidden_size up to 1024 on a device of 8 XCDs x 32 CUs; PIMHIP_ERR_UNSUPPORTED
 * otherwise).  A call with seq_len 1 runs the fused step launch in every mode.
 * Automatic mode measures: the first pimhip_lstm_forward of a plan with a sequence length in [2^b, 2^(b+1)) that is issued
 * outside a graph capture runs the call under every mode that takes it (a few runs each, timed with HIP events: that
 * call synchronises its stream and costs a few times its usual duration), and the plan keeps the fastest for that range of
 * lengths; as the reference does with its two libraries on the first inference
 * (runtime/source/executor/stream_executor.cpp:312-339).  Until then (calls inside a capture, or after
 * pimhip_lstm_plan_set_measure(plan, 0)) thresholds measured once on MI355X choose: 4 for bidirectional layers and for a
 * single unidirectional layer when the sequence is long enough to pay for it, 4 or 2 for unidirectional stacks, 1 where
 * neither fits. */
int pimhip_lstm_plan_set_mode(PimHipLstmPlan* plan, int mode);

/* No counterpart in the reference beyond the above.  enabled == 0: automatic mode stops measuring and forgets what it
 * measured (thresholds choose); != 0 (the default): it measures as described.  pimhip_lstm_plan_measured_mode: the mode
 * automatic mode uses for sequences of seq_len (>= 2) steps, 0 if that range of lengths has not been measured yet. */
int pimhip_lstm_plan_set_measure(PimHipLstmPlan* plan, int enabled);
int pimhip_lstm_plan_measured_mode(PimHipLstmPlan* plan, int64_t seq_len, int* mode);

/* No counterpart in aten::lstm.  Layers first_residual_layer .. num_layers - 1 of a unidirectional stack hand up and
 * return out_t = h_t + in_t (fp16, one rounding) instead of h_t, in_t being the layer's own input: the wiring of the GNMT
 * encoder and decoder, which the reference runs as one executeAtenLSTM1 and one executeAtenAdd per layer
 * (aten_ops_executor.cpp:2135-2307, :43-179).  hn / cn stay the layers' own h and c.  Such a layer's input width must equal
 * hidden_size.  first_residual_layer >= num_layers switches it off (the default).  A stack then still runs as one
 * pipeline launch where pimhip_lstm_forward would use one without the sums. */
int pimhip_lstm_plan_set_residual(PimHipLstmPlan* plan, int first_residual_layer);

/* The dense input projection of one LSTM layer over all time steps, the only MFMA kernel of the path:
 * out[T, n_out] (fp32) = x[T, in] (fp16) . w[n_out, in]^T (fp16) + bias[n_out] (fp32, may be NULL). */
int pimhip_input_projection(void* out, const void* x, const void* w, const void* bias, int64_t seq_len,
                            int64_t in_w, int64_t n_out, void* stream);

/* The same product with the weight re-laid out once in the matrix cores' fragment order, which is what an LSTM plan
 * does with the w_ih of its batched layers at creation (it takes the place of the MIOpen weight packing,
 * model_builder.cpp:226-319): pimhip_projection_packed_bytes gives the size of the packed copy,
 * pimhip_pack_projection_weight fills it from w[n_out, in_w] (row-major, dense), and
 * pimhip_input_projection_packed computes out[T, n_out] from it (the same exact products as pimhip_input_projection,
 * summed in a fixed order that may differ from its).
 * They have no counterpart in the reference; they are exported for callers that batch the projection themselves. */
int pimhip_projection_packed_bytes(int64_t in_w, int64_t n_out, uint64_t* bytes);
int pimhip_pack_projection_weight(void* packed, const void* w, int64_t in_w, int64_t n_out, void* stream);
int pimhip_input_projection_packed(void* out, const void* x, const void* packed, const void* bias, int64_t seq_len,
                                   int64_t in_w, int64_t n_out, void* stream);

/* No counterpart in the reference (the PIM SDK's PimExecuteGemm reports nothing either, aten_ops.cpp:659).
 * A reducing block of a sliced I_X_W product that gave up waiting for partial sums (a bounded wait: other work kept part
 * of the GPU from running the blocks that produce them) computes them itself; nothing is left undefined.  For a caller that
 * wants to know, after synchronising the stream: *gave_up gets bit 0 if a product of pimhip_execute_gemv / _bmm on `stream`
 * did so since the workspace was last put in order, bit 1 if one of pimhip_execute_gemv_static on this GPU did;
 * pimhip_gemv_fallbacks gives the number of such events so far on `stream` plus those of the static entry point.
 * pimhip_set_gemv_spin_limit sets the number of polls per record for the current GPU (default 2^22, seconds); with 0 a
 * reducing block gives up without polling, which is how tests force the condition while every kernel still ends. */
int pimhip_gemv_status(void* stream, int* gave_up);
int pimhip_gemv_fallbacks(void* stream, uint64_t* events);
int pimhip_set_gemv_spin_limit(unsigned int spin_limit);

/* ---- decoder step ---------------------------------------------------------------------------- */

typedef struct PimHipDecoderPlan PimHipDecoderPlan;

/* One launch for one step of a GNMT-style decoder stack.  Replaces, for that step, the chain of operator calls the
 * reference's interpreter makes in its decoder loop: executeAtenLSTM1 with seq_len == 1 once per layer
 * (aten_ops_executor.cpp:2135-2307; miopen_ops_executor.cpp:170-228 for where hy / cy / out land), executeAtenBmm for the
 * attention context (aten_ops_executor.cpp:668-747), executeAtenAdd for the residual sums (aten_ops_executor.cpp:43-179)
 * and executeAtenAddmm for the classifier (aten_ops_executor.cpp:181-216):
 *
 *     ctx    = att[1, S] . enc[S, H]                               (or ctx_in)
 *     y_0    = lstm_0(x)            or lstm_0(cat(x, ctx)) when first_takes_context
 *     y_k    = lstm_k(cat(in_k, ctx)),  in_1 = out_0, in_{k+1} = out_k          (k >= 1)
 *     out_k  = y_k + in_k  for k >= first_residual_layer (in_0 = x), else y_k
 *     logits = classifier_w[vocab, H] . out_last + classifier_b                 (when classifier_w is given)
 *
 * The whole GNMT decoder step is (4 layers, first_takes_context 0, first_residual_layer 2, classifier); where other
 * operators sit between layer 0 and the context (the attention scores), layer 0 stays a pimhip_lstm_forward call and
 * the rest of the step is a plan with (3 layers, first_takes_context 1, first_residual_layer 1).
 *   params: host array of device pointers in LibTorch order per layer (w_ih [4H, in_w], w_hh [4H, H], then b_ih, b_hh
 *           [4H] when has_biases), gate order (i, f, g, o); in_w = input_size for a plain first layer, 2H for every layer
 *           that takes cat(in, ctx).  num_layers 1..4, hidden_size a multiple of 8 up to 1024, input_size a multiple
 *           of 8 (== hidden_size when first_takes_context or first_residual_layer == 0).
 * The plan keeps the weight pointers (they must outlive it), pre-adds the biases and owns a small exchange buffer.
 * Runs on `stream` and synchronises it. */
int pimhip_decoder_plan_create(PimHipDecoderPlan** plan, const void* const* params, int n_params, int has_biases,
                               int num_layers, int first_takes_context, int first_residual_layer, int64_t input_size,
                               int64_t hidden_size, const void* classifier_w, const void* classifier_b, int64_t vocab,
                               void* stream);

int pimhip_decoder_plan_destroy(PimHipDecoderPlan* plan);

/* Once per sentence (whenever the encoder outputs change): enc [enc_len, H], row-major and dense.  The context columns
 * of every layer's W_ih are multiplied with enc here, once (enc . W_ih[:, H:2H]^T, fp32, on the matrix cores), because
 * W_ih[:, H:2H] . (att . enc) = (W_ih[:, H:2H] . enc^T) . att: a step then reads enc_len values per gate row instead of
 * streaming those H columns, and needs no context vector.  The plan keeps the pointer (enc must stay valid and unchanged
 * until the next call; it is read again only by steps that store the context).  Enqueues on `stream`; a call that needs
 * a larger buffer than the plan has synchronises the stream and allocates (not on a capturing stream). */
int pimhip_decoder_plan_set_encoder(PimHipDecoderPlan* plan, const void* enc, int64_t enc_len, void* stream);

/* One step.  x [input_size]; att [enc_len], the attention weights over the encoder outputs given to
 * pimhip_decoder_plan_set_encoder, or instead ctx_in [H], a context computed elsewhere (its columns are then streamed);
 * h_prev, c_prev, hn, cn, layer_outs: host arrays of num_layers device pointers to [H] vectors (the rows of a state
 * buffer, for instance); layer_outs, or any entry of it, may be NULL, otherwise entry k receives out_k; the context is
 * also stored to the n_ctx_outs (0..4) buffers of ctx_outs; logits [vocab].  hn[k] / cn[k] may be the buffers
 * h_prev[k] / c_prev[k] were read from (a one-layer plan without a classifier excepted); no other output may alias an
 * input.  All blocks of the launch have to be resident at once, so the call is ordered like a sequence call of
 * pimhip_lstm_forward against the device's other such launches, and steps sharing a plan must be ordered on one stream.
 * h_prev, c_prev and x 16-byte aligned.
 * Records one kernel.  Every wait inside is bounded (a poll count and one second).  When one gives up because part of the
 * grid was kept from running, the block that waited computes the missing values itself, in the order their owner would
 * have (the step's results are bit for bit what they would have been), and a block that cannot know whether every other
 * block has read the previous state yet keeps its new state in the plan's memory until the last block of the launch
 * stores it to hn / cn: the in-place update stays safe.  Slower (milliseconds when most of the grid is missing), never
 * undefined; pimhip_decoder_plan_fallbacks counts the events. */
int pimhip_decoder_step(PimHipDecoderPlan* plan, const void* x, const void* att, const void* ctx_in,
                        const void* const* h_prev, const void* const* c_prev, void* const* hn,
                        void* const* cn, void* const* layer_outs, void* const* ctx_outs, int n_ctx_outs, void* logits,
                        void* stream);

/* Always PIMHIP_OK for a valid plan: no step of this plan leaves an undefined result (kept for callers of the earlier
 * interface, where a wait that gave up was an error). */
int pimhip_decoder_plan_status(PimHipDecoderPlan* plan);
/* The poll limit of the waits inside a step (default 2^22; 0: a wait gives up at its first look, which tests use). */
int pimhip_decoder_plan_set_spin_limit(PimHipDecoderPlan* plan, unsigned int spin_limit);
/* No counterpart in the reference.  *events: how many times a wait inside a step of this plan has given up so far (as far
 * as the host has seen: ask after synchronising the stream; counted per step that had one, when the next step is issued
 * outside a graph capture or here); *patient (may be null): 1 while waits run to the plan's poll limit, 0 once, after
 * the third event, every wait of the plan's steps gives up after 4096 polls. */
int pimhip_decoder_plan_fallbacks(PimHipDecoderPlan* plan, uint64_t* events, int* patient);

/* ---- mixture-of-experts feed-forward step ----------------------------------------------------- */

typedef struct PimHipMoePlan PimHipMoePlan;

/* One launch for a token's pass through a top-1 mixture-of-experts feed-forward block (the Switch Transformer's):
 *
 *     logits = router_w[E, d_model] . x (+ router_b)      e = argmax(logits)   (first maximum, logits rounded to fp16)
 *     hidden = act(w1[e][d_ff, d_model] . x + b1[e])                           (rounded to fp16)
 *     y      = w2[e][d_model, d_ff] . hidden + b2[e]      (times softmax(logits)[e] when scale_by_router_prob)
 *
 * Replaces three customAtenAddmm / atenLinear calls (aten_ops.cpp:609-758, :304-307) and the host's choice of the
 * expert between them, which costs the reference's interpreter a stream synchronisation and a read-back per token; here
 * the choice is made on the GPU and only expert e's weights are read.
 *   w1, b1, w2, b2: host arrays of E device pointers (b1 / b2 may be null arrays: no bias); all weights row-major, dense,
 *   fp16, 16-byte aligned.  E <= 64; d_model <= 2048 and d_ff <= 4096, multiples of 8 (PIMHIP_ERR_UNSUPPORTED
 *   otherwise: three pimhip_execute_gemv calls serve any size); act as in pimhip_execute_gemv.
 * The plan keeps the pointers (the weights must outlive it) and owns a 32 KiB exchange buffer.  The workgroups of a step
 * (at most 256) exchange the hidden values among themselves and have to be resident together; the library orders the step
 * against its other such launches (pimhip_lstm_forward, pimhip_decoder_step), and steps sharing a plan must be ordered
 * on one stream. */
int pimhip_moe_plan_create(PimHipMoePlan** plan, const void* router_w, const void* router_b, const void* const* w1,
                           const void* const* b1, const void* const* w2, const void* const* b2, int num_experts,
                           int64_t d_model, int64_t d_ff, int act, int scale_by_router_prob, void* stream);
int pimhip_moe_plan_destroy(PimHipMoePlan* plan);

/* x [d_model] (16-byte aligned), y [d_model]; router_logits [E] fp16 and expert [1] int32 are device pointers or null.
 * Records one kernel.  Every wait inside is bounded, and a wait that gives up (other work kept part of the GPU from running
 * the step's workgroups together) costs time, not the result: the workgroups that waited in vain compute the missing
 * hidden values themselves, inside the same launch, and y is what it would have been.  Later steps do the same from the
 * start until a step issued outside a graph capture has put the exchange back in order (it synchronises the stream then);
 * after the third such event the plan stops exchanging for good (about 25 times slower per step, still one launch). */
int pimhip_moe_ffn_step(PimHipMoePlan* plan, const void* x, void* y, void* router_logits, int* expert, void* stream);

/* Always PIMHIP_OK for a valid plan: no step of this plan leaves an undefined result (kept for callers of the earlier
 * interface, where a wait that gave up was an error). */
int pimhip_moe_plan_status(PimHipMoePlan* plan);

/* No counterpart in the reference.  *events: how many times a wait inside a step of this plan has given up so far (as far
 * as the host has seen: ask after synchronising the stream); *exchanging (may be null): 1 while steps still exchange
 * hidden values between workgroups, 0 once the plan has gone over to the self-sufficient mode for good. */
int pimhip_moe_plan_fallbacks(PimHipMoePlan* plan, uint64_t* events, int* exchanging);

/* Polls of one wait before it gives up (default 2^22, roughly seconds).  Tests pass 0 so that every wait whose first look
 * fails gives up at once: every kernel still ends by itself. */
int pimhip_moe_plan_set_spin_limit(PimHipMoePlan* plan, unsigned int spin_limit);

/* ---- RNN-transducer decoding step --------------------------------------------------------------- */

typedef struct PimHipRnntPlan PimHipRnntPlan;

/* One launch for one (t, u) step of an RNN-transducer's greedy decoding loop: the prediction network's LSTM cells at
 * seq_len 1 and the joint network.  Replaces, per iteration of that loop, executeAtenLSTM1 with seq_len == 1
 * (aten_ops_executor.cpp:2135-2307) and the joint network's executeAtenAddmm calls (aten_ops_executor.cpp:181-216), the
 * first of which RemoveCatForAddmm has split into two dependent products over the two halves of the concatenated input
 * (compiler/source/frontend/optimizer/remove_cat_for_addmm.cpp:46-191):
 *
 *     h_l, c_l = lstm_cell_l(l == 0 ? x : h_{l-1}; h_prev_l, c_prev_l)                    l < num_layers
 *     hidden   = relu(joint_w1[joint_size, enc_size + H] . cat(f, g) + joint_b1)          g = h of the last layer
 *     logits   = joint_w2[vocab, joint_size] . hidden + joint_b2
 *
 *   params: host array of device pointers in LibTorch order per layer (w_ih [4H, in_w], w_hh [4H, H], then b_ih, b_hh
 *           [4H] when has_biases), gate order (i, f, g, o); in_w = input_size for the first layer, H above it.
 *   num_layers 1..4; hidden_size and input_size multiples of 8 up to 1024; enc_size and joint_size multiples of 8 up to
 *   2048; one workgroup per eight hidden units of a layer, per eight joint units and per eight symbols, at most 256 in all
 *   (RNNT: 2 x 40 + 64 + 4 = 148); PIMHIP_ERR_UNSUPPORTED otherwise (pimhip_lstm_forward, pimhip_execute_gemv_cat2 and
 *   pimhip_execute_gemv serve any size).  Weights row-major, dense, fp16, 16-byte aligned.
 * The plan keeps the weight pointers (they must outlive it), pre-adds the biases and owns a small exchange buffer.  Runs
 * on `stream` and synchronises it. */
int pimhip_rnnt_plan_create(PimHipRnntPlan** plan, const void* const* params, int n_params, int has_biases, int num_layers,
                            int64_t input_size, int64_t hidden_size, const void* joint_w1, const void* joint_b1,
                            int64_t joint_size, int64_t enc_size, const void* joint_w2, const void* joint_b2, int64_t vocab,
                            void* stream);
int pimhip_rnnt_plan_destroy(PimHipRnntPlan* plan);

/* One step.  x [input_size] (the embedding of the last symbol), h_prev, c_prev, hn, cn [num_layers, H], f [enc_size] (the
 * encoder's output for frame t), logits [vocab]; joint_hidden [joint_size] or null.  run_prediction == 0 is the step after
 * a blank, where only the frame has changed: the prediction network does not run, g = h_prev of the last layer, and x,
 * c_prev, hn, cn are not touched (they may be null).  hn / cn must not overlap h_prev / c_prev (keep two state buffers and
 * swap them).
 * Records one kernel, so steps can be recorded into a HIP graph.  All workgroups of the launch have to be resident at
 * once: the call is ordered like a sequence call of pimhip_lstm_forward against the device's other such launches, and
 * steps sharing a plan must be ordered on one stream.  Every wait inside is bounded, and a wait that gives up costs time,
 * not the result: the workgroup that waited in vain computes the vector it waited for by itself, inside the same launch,
 * with the same sums, and the outputs are what they would have been.  Later steps do the same from the start until a step
 * issued outside a graph capture has put the exchange back in order (it synchronises the stream then); after the third
 * such event the plan stops exchanging for good (slower, still one launch). */
int pimhip_rnnt_step(PimHipRnntPlan* plan, const void* x, const void* h_prev, const void* c_prev, const void* f, void* hn,
                     void* cn, void* logits, void* joint_hidden, int run_prediction, void* stream);

/* The whole greedy decoding loop over one utterance in one launch: what the reference interprets operator by operator per
 * iteration of prim::Loop (runtime/source/executor/op_executor/prim_ops_executor.cpp:820-875: executeAtenLSTM1 with
 * seq_len == 1, the joint network's executeAtenAddmm calls and executeAtenArgmax, aten_ops_executor.cpp:520-560, whose
 * result the host reads before the next iteration).
 *
 *     t = 0; g, state = prediction(x0, (h0, c0))          (run_prediction_first == 0: g = h0 of the last layer as it is)
 *     while t < n_frames and fewer than max_symbols emitted:
 *         k = argmax(logits(enc[t], g))                    (fp16 logits; the first maximum, a NaN counting as the largest)
 *         if k == blank: t += 1
 *         else: symbols[n++] = k; g, state = prediction(embedding[k], state);
 *               after max_symbols_per_frame symbols of one frame: t += 1
 *
 *   enc [n_frames, enc_size], embedding [embedding_rows >= vocab, input_size] (row k: the prediction network's input after
 *   symbol k), x0 [input_size] (its input before any symbol), h0 / c0 [num_layers, H] or null (zeros), hn / cn the same
 *   shape or null, not overlapping h0 / c0; symbols [max_symbols] int32; result [8] int32: symbols emitted, frames
 *   consumed, steps taken, 1 if one workgroup had to decode alone, 1 if the last symbol has not been fed to the prediction
 *   network yet (hn / cn are the state before it), the last symbol (-1: none), 0, 0.  All device memory; fp16 tensors
 *   dense and 16-byte aligned.  vocab <= 512 (PIMHIP_ERR_UNSUPPORTED otherwise: drive pimhip_rnnt_step from the host).
 * Symbols and final state equal, bit for bit, those of the same loop driven from the host through pimhip_rnnt_step.
 * Asynchronous; records three kernels, so it can be recorded into a HIP graph.  Residency, ordering and the plan's stream
 * as for pimhip_rnnt_step.  Every wait inside is bounded; when one gives up, one workgroup decodes the utterance again from
 * its start by itself inside the same launch (slower, the same result), and the event counts for the plan like a step's. */
int pimhip_rnnt_greedy_decode(PimHipRnntPlan* plan, const void* enc, int64_t n_frames, const void* embedding, int64_t embedding_rows,
                              const void* x0, const void* h0, const void* c0, int run_prediction_first, int blank,
                              int max_symbols_per_frame, int64_t max_symbols, int32_t* symbols, int32_t* result, void* hn, void* cn,
                              void* stream);

/* No counterpart in the reference.  As pimhip_moe_plan_fallbacks / pimhip_moe_plan_set_spin_limit. */
int pimhip_rnnt_plan_fallbacks(PimHipRnntPlan* plan, uint64_t* events, int* exchanging);
int pimhip_rnnt_plan_set_spin_limit(PimHipRnntPlan* plan, unsigned int spin_limit);

#ifdef __cplusplus
}
#endif

#endif /* PIMHIP_H_ */
