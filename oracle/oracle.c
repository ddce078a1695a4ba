/*
 * oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C CPU restatement of the reference's fp16 GEMV / LSTM hot path, used only by tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg as the checker for the HIP kernels.  Nothing in
 * pimaicompiler_amd/ may call it.
 *
 * What follows what (paths relative to the reference tree):
 *   oracle_gemm_broadcast   gemmBroadcast, line by line      runtime/source/executor/utils/utils.cpp:293-371
 *   oracle_get_gemm_type    getGemmType, line by line        runtime/source/executor/utils/utils.cpp:373-396
 *   oracle_gemv_mv / _vm    y = A.x + b / x.A + b, ReLU last runtime/include/executor/op_executor/custom_ops.h:216-381
 *                           (the operation customAtenAddmm requests from the PIM SDK,
 *                            runtime/source/executor/op_executor/aten_ops.cpp:626-694; alpha = 1, beta = 0 there)
 *   oracle_add              custom_add (element-wise, row broadcast) runtime/include/executor/op_executor/custom_ops.h:383-433
 *   oracle_dot              VV branch of customAtenMatmul    runtime/source/executor/op_executor/aten_ops.cpp:841-882
 *   oracle_lstm             at::lstm as atenLstm1/2 call it  runtime/source/executor/op_executor/aten_ops.cpp:328-344
 *                           with the parameter order of      runtime/source/builder/model_builder.cpp:158-224
 *   oracle_lstm_pack_miopen reArangeLstmWeights              runtime/source/builder/model_builder.cpp:226-319
 *
 * The arithmetic of the GEMV lives in the un-vendored PIM SDK (SAITPublic/PIMLibrary, no version pinned) and
 * that of the LSTM in LibTorch (unpinned); the reference's own tests define the GEMV result as at::matmul
 * within atol 1e-3 / rtol 1e-5 (runtime/unit-tests/custom_op_ut.cpp:45,67,109,146).  This file therefore
 * restates the published mathematics: exact fp16 products, accumulation in double, one rounding to fp16 where
 * the interface stores fp16 (GEMV outputs; h_t and the final c of the LSTM).
 *
 * Pinning (tests/test_oracle.py): LibTorch-CPU golden vectors in tests/golden/ (at::addmm, at::matmul,
 * at::lstm on seeded inputs), closed forms (zero input, one-hot input, identity weight, zero-weight LSTM),
 * VM/MV transposition symmetry, bidirectional = time reversal, multi-layer = composition, pack/unpack
 * round trip.  oracle_gemm_broadcast / oracle_get_gemm_type have no reference test or fixture: they are a
 * line-by-line restatement checked against hand-derived cases only.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- IEEE binary16 <-> double -------------------------------------------------------------- */
static double half_to_double(uint16_t h)
{
    const int sign = (h >> 15) & 1;
    const int exp = (h >> 10) & 0x1f;
    const int man = h & 0x3ff;
    double v;
    if (exp == 0)
        v = ldexp((double)man, -24);
    else if (exp == 31)
        v = man ? NAN : INFINITY;
    else
        v = ldexp((double)(man | 0x400), exp - 25);
    return sign ? -v : v;
}

/* Round to nearest, ties to even, directly from double (no double rounding through float). */
static uint16_t double_to_half(double d)
{
    uint16_t sign = 0;
    if (signbit(d)) {
        sign = 0x8000;
        d = -d;
    }
    if (isnan(d)) return (uint16_t)(sign | 0x7e00);
    if (d >= 65520.0) return (uint16_t)(sign | 0x7c00); /* rounds to infinity */
    if (d < ldexp(1.0, -25)) return sign;               /* below half of the smallest subnormal */
    int e;
    (void)frexp(d, &e); /* d = f * 2^e, f in [0.5, 1) */
    int exp = e - 1;    /* d in [2^exp, 2^(exp+1)) */
    if (exp < -14) exp = -14;
    /* quantum = 2^(exp-10) */
    const double q = ldexp(d, 10 - exp);
    double r = nearbyint(q); /* default rounding mode: to nearest even */
    int biased = exp + 15;
    if (exp == -14 && r < 1024.0) {
        return (uint16_t)(sign | (uint16_t)r); /* subnormal (or zero) */
    }
    if (r >= 2048.0) {
        r = 1024.0;
        biased += 1;
    }
    if (biased >= 31) return (uint16_t)(sign | 0x7c00);
    return (uint16_t)(sign | (biased << 10) | ((uint16_t)r & 0x3ff));
}

double oracle_half_to_double(uint16_t h) { return half_to_double(h); }
uint16_t oracle_double_to_half(double d) { return double_to_half(d); }

/* ---- shape logic --------------------------------------------------------------------------- */
/* A tiny vector<int64_t> with the three operations gemmBroadcast uses. */
typedef struct {
    int64_t v[8];
    int n;
} shape_t;

static void shape_insert(shape_t* s, int pos, int64_t val)
{
    for (int i = s->n; i > pos; --i) s->v[i] = s->v[i - 1];
    s->v[pos] = val;
    s->n++;
}

/* Return: 0 ok, 1 the reference would abort (DLOG(FATAL)), 2 the reference would index out of range. */
static int broadcast_rec(shape_t* s1, shape_t* s2)
{
    const int dim1 = s1->n, dim2 = s2->n;
    if (dim1 == dim2) { /* utils.cpp:299-310 */
        shape_t t1 = {{0}, 0}, t2 = {{0}, 0};
        for (int i = 0; i < 4; i++) {
            if (i < dim1) {
                t1.v[t1.n++] = s1->v[i];
                t2.v[t2.n++] = s2->v[i];
            } else {
                shape_insert(&t1, 0, 1);
                shape_insert(&t2, 0, 1);
            }
        }
        *s1 = t1;
        *s2 = t2;
        return 0;
    } else if (dim1 < dim2) { /* utils.cpp:311-334 */
        const int num = dim2 - dim1;
        if (num == 1) {
            if (s1->v[0] == s2->v[0])
                shape_insert(s1, 1, 1);
            else
                shape_insert(s1, 0, 1);
            return broadcast_rec(s1, s2);
        } else if (num == 2) {
            if (s1->v[0] == s2->v[0]) {
                shape_insert(s1, 1, 1);
                shape_insert(s1, 1, 1);
            } else if (s1->v[0] == s2->v[1]) {
                shape_insert(s1, 1, 1);
                shape_insert(s1, 0, 1);
            } else {
                if (dim1 < 2) return 2; /* reads shape1[1] of a rank-1 shape */
                if (s1->v[1] == s2->v[2]) {
                    shape_insert(s1, 0, 1);
                    shape_insert(s1, 0, 1);
                }
            }
            return 0;
        }
        return 1;
    } else { /* utils.cpp:335-370 */
        const int num = dim1 - dim2;
        if (num == 1) {
            if (dim2 < 2) { /* reads shape2[dim2 - 2] = shape2[-1]; any value but a match appends */
                s2->v[s2->n++] = 1;
            } else if (s1->v[dim1 - 1] == s2->v[dim2 - 2]) {
                shape_insert(s2, 0, 1);
            } else {
                s2->v[s2->n++] = 1;
            }
            return broadcast_rec(s1, s2);
        } else if (num == 2) {
            if (dim1 < 4 || dim2 < 2) return 2; /* reads shape1[3] / shape2[1] */
            if (s1->v[3] == s2->v[1])
                s2->v[s2->n++] = 1;
            else
                shape_insert(s2, 0, 1);
            if (s1->v[0] == s2->v[0])
                shape_insert(s2, 1, 1);
            else
                shape_insert(s2, 0, 1);
            return 0;
        } else if (num == 3) {
            const int64_t tmp = s2->v[0];
            *s2 = *s1;
            if (tmp == s1->v[3]) {
                s2->v[2] = tmp;
                s2->v[3] = 1;
            } else {
                s2->v[2] = 1;
                s2->v[3] = tmp;
            }
            return 0;
        }
        return 1;
    }
}

int oracle_gemm_broadcast(int64_t* shape1, int* rank1, int64_t* shape2, int* rank2)
{
    shape_t a = {{0}, 0}, b = {{0}, 0};
    if (*rank1 < 1 || *rank1 > 4 || *rank2 < 1 || *rank2 > 4) return 1;
    for (int i = 0; i < *rank1; ++i) a.v[a.n++] = shape1[i];
    for (int i = 0; i < *rank2; ++i) b.v[b.n++] = shape2[i];
    const int rc = broadcast_rec(&a, &b);
    if (rc != 0) return rc;
    for (int i = 0; i < a.n; ++i) shape1[i] = a.v[i];
    for (int i = 0; i < b.n; ++i) shape2[i] = b.v[i];
    *rank1 = a.n;
    *rank2 = b.n;
    return 0;
}

/* Returns the integer of GEMM_TYPE {UNKNOW, VV, MV, VM, MM} (runtime/include/executor/utils/utils.h:30-36): VV 1, MV 2,
 * VM 3, MM 4.  utils.cpp:373-396. */
int oracle_get_gemm_type(const int64_t* self_shape, const int64_t* other_shape)
{
    if (self_shape[0] == 1 && self_shape[1] == 1 && other_shape[0] == 1 && other_shape[1] == 1) {
        int self_is_vector = 0, other_is_vector = 0;
        if (self_shape[2] != 1) self_is_vector++;
        if (self_shape[3] != 1) self_is_vector++;
        if (other_shape[2] != 1) other_is_vector++;
        if (other_shape[3] != 1) other_is_vector++;
        if (self_is_vector == 1 && other_is_vector == 1) return 1;
        if (self_is_vector == 1 && other_is_vector == 2) return 3; /* VM */
        if (self_is_vector == 2 && other_is_vector == 1) return 2; /* MV */
        return 4;
    }
    return 4;
}

/* ---- GEMV family ---------------------------------------------------------------------------- */
static uint16_t epilogue(double acc, const uint16_t* bias, int64_t i, int relu)
{
    if (bias) acc += half_to_double(bias[i]);
    if (relu && acc < 0.0) acc = 0.0;
    return double_to_half(acc);
}

/* y[n] = act(sum_k W[n*ldw + k] * x[k] + bias[n]) */
void oracle_gemv_mv(const uint16_t* W, const uint16_t* x, const uint16_t* bias, uint16_t* y, int64_t N, int64_t K,
                    int64_t ldw, int relu)
{
    double* xd = (double*)malloc(sizeof(double) * (size_t)(K > 0 ? K : 1));
    for (int64_t k = 0; k < K; ++k) xd[k] = half_to_double(x[k]);
    for (int64_t n = 0; n < N; ++n) {
        double acc = 0.0;
        const uint16_t* w = W + n * ldw;
        for (int64_t k = 0; k < K; ++k) acc += half_to_double(w[k]) * xd[k];
        y[n] = epilogue(acc, bias, n, relu);
    }
    free(xd);
}

/* y[n] = act(sum_k x[k] * A[k*lda + n] + bias[n]) */
void oracle_gemv_vm(const uint16_t* x, const uint16_t* A, const uint16_t* bias, uint16_t* y, int64_t K, int64_t N,
                    int64_t lda, int relu)
{
    double* acc = (double*)calloc((size_t)(N > 0 ? N : 1), sizeof(double));
    for (int64_t k = 0; k < K; ++k) {
        const double xv = half_to_double(x[k]);
        const uint16_t* a = A + k * lda;
        for (int64_t n = 0; n < N; ++n) acc[n] += xv * half_to_double(a[n]);
    }
    for (int64_t n = 0; n < N; ++n) y[n] = epilogue(acc[n], bias, n, relu);
    free(acc);
}

void oracle_dot(const uint16_t* a, const uint16_t* b, uint16_t* y, int64_t K)
{
    double acc = 0.0;
    for (int64_t k = 0; k < K; ++k) acc += half_to_double(a[k]) * half_to_double(b[k]);
    y[0] = double_to_half(acc);
}

/* c[m][n] = a[m][n] + b, b being [m][n] or one row [n] (custom_add, custom_ops.h:383-433; alpha is ignored there):
 * the exact sum rounded once to fp16. */
void oracle_add(const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t m, int64_t n, int b_broadcast)
{
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j)
            c[i * n + j] = double_to_half(half_to_double(a[i * n + j]) + half_to_double(b[b_broadcast ? j : i * n + j]));
}

/* The same MV product with float storage and float accumulation: the scalar fp32 figure beside the fp16 one
 * in the CPU baseline. */
void oracle_gemv_mv_f32(const float* W, const float* x, const float* bias, float* y, int64_t N, int64_t K)
{
    for (int64_t n = 0; n < N; ++n) {
        float acc = 0.0f;
        const float* w = W + n * K;
        for (int64_t k = 0; k < K; ++k) acc += w[k] * x[k];
        y[n] = acc + (bias ? bias[n] : 0.0f);
    }
}

/* ---- LSTM ----------------------------------------------------------------------------------- */
static double sigmoid_d(double v) { return 1.0 / (1.0 + exp(-v)); }

/* One (layer, direction): x [T, I] -> y rows at y + t * y_stride, state h0/c0 -> hn/cn, all fp16 at the
 * interface; gate order (i, f, g, o). */
static void lstm_cell_sequence(const uint16_t* x, int64_t T, int64_t I, int64_t H, const uint16_t* w_ih,
                               const uint16_t* w_hh, const uint16_t* b_ih, const uint16_t* b_hh, const uint16_t* h0,
                               const uint16_t* c0, int reverse, uint16_t* y, int64_t y_stride, uint16_t* hn,
                               uint16_t* cn)
{
    double* h = (double*)malloc(sizeof(double) * (size_t)H);
    double* c = (double*)malloc(sizeof(double) * (size_t)H);
    double* a = (double*)malloc(sizeof(double) * (size_t)(4 * H));
    double* xt = (double*)malloc(sizeof(double) * (size_t)I);
    double* wih = (double*)malloc(sizeof(double) * (size_t)(4 * H * I));
    double* whh = (double*)malloc(sizeof(double) * (size_t)(4 * H * H));
    for (int64_t i = 0; i < 4 * H * I; ++i) wih[i] = half_to_double(w_ih[i]);
    for (int64_t i = 0; i < 4 * H * H; ++i) whh[i] = half_to_double(w_hh[i]);
    for (int64_t j = 0; j < H; ++j) {
        h[j] = half_to_double(h0[j]);
        c[j] = half_to_double(c0[j]);
    }
    for (int64_t s = 0; s < T; ++s) {
        const int64_t t = reverse ? (T - 1 - s) : s;
        for (int64_t k = 0; k < I; ++k) xt[k] = half_to_double(x[t * I + k]);
        for (int64_t r = 0; r < 4 * H; ++r) {
            double acc = 0.0;
            const double* wi = wih + r * I;
            for (int64_t k = 0; k < I; ++k) acc += wi[k] * xt[k];
            const double* wh = whh + r * H;
            for (int64_t k = 0; k < H; ++k) acc += wh[k] * h[k];
            if (b_ih) acc += half_to_double(b_ih[r]);
            if (b_hh) acc += half_to_double(b_hh[r]);
            a[r] = acc;
        }
        for (int64_t j = 0; j < H; ++j) {
            const double ig = sigmoid_d(a[j]), fg = sigmoid_d(a[H + j]), gg = tanh(a[2 * H + j]),
                         og = sigmoid_d(a[3 * H + j]);
            c[j] = fg * c[j] + ig * gg;
            const uint16_t hb = double_to_half(og * tanh(c[j]));
            y[t * y_stride + j] = hb;
            h[j] = half_to_double(hb); /* h is fp16 at the interface: the next step sees the rounded value */
        }
    }
    for (int64_t j = 0; j < H; ++j) {
        hn[j] = double_to_half(h[j]);
        cn[j] = double_to_half(c[j]);
    }
    free(h); free(c); free(a); free(xt); free(wih); free(whh);
}

/* params: LibTorch order per layer then direction: w_ih, w_hh[, b_ih, b_hh] (model_builder.cpp:185-213).
 * x [T, I]; h0, c0, hn, cn [L*D, H] ordered (l0 fwd, l0 bwd, l1 fwd, ...); y [T, D*H]. */
void oracle_lstm(const uint16_t* x, int64_t T, int64_t I, int64_t H, int num_layers, int bidirectional,
                 int has_biases, const uint16_t* const* params, const uint16_t* h0, const uint16_t* c0, uint16_t* y,
                 uint16_t* hn, uint16_t* cn)
{
    const int D = bidirectional ? 2 : 1;
    const int per_cell = has_biases ? 4 : 2;
    const int64_t width = (int64_t)D * H;
    uint16_t* buf[2];
    buf[0] = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(T * width > 0 ? T * width : 1));
    buf[1] = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(T * width > 0 ? T * width : 1));
    const uint16_t* in = x;
    int64_t in_w = I;
    for (int l = 0; l < num_layers; ++l) {
        uint16_t* out = (l == num_layers - 1) ? y : buf[l & 1];
        for (int d = 0; d < D; ++d) {
            const int ci = l * D + d;
            const uint16_t* const* p = params + (size_t)ci * per_cell;
            lstm_cell_sequence(in, T, in_w, H, p[0], p[1], has_biases ? p[2] : NULL, has_biases ? p[3] : NULL,
                               h0 + (int64_t)ci * H, c0 + (int64_t)ci * H, d, out + (int64_t)d * H, width,
                               hn + (int64_t)ci * H, cn + (int64_t)ci * H);
        }
        in = out;
        in_w = width;
    }
    free(buf[0]);
    free(buf[1]);
}

/* reArangeLstmWeights (model_builder.cpp:226-319): one contiguous fp16 buffer; for every layer the four gate
 * chunks of each tensor are stored in the order (0, 1, 3, 2); all weights first (per layer: w_ih fwd,
 * [w_ih bwd,] w_hh fwd[, w_hh bwd]), then all biases in the same pattern.  sizes[i] = element count of
 * params[i].  direction 0: pack params -> buffer; direction 1: unpack buffer -> params. */
void oracle_lstm_pack_miopen(uint16_t* const* params, const int64_t* sizes, int num_layers, int bidirectional,
                             int has_biases, uint16_t* buffer, int unpack)
{
    static const int perm[4] = {0, 1, 3, 2};
    const int D = bidirectional ? 2 : 1;
    const int per_cell = has_biases ? 4 : 2;
    const int num_offset = per_cell * D;          /* tensors per layer */
    const int param_num = per_cell * num_layers * D;
    int64_t offset = 0;
    for (int pass = 0; pass < (has_biases ? 2 : 1); ++pass) {
        const int start = pass * 2; /* 0: weights, 2: biases */
        for (int num = start; num < param_num; num += num_offset) {
            for (int index_offset = 0; index_offset < 2; ++index_offset) {
                for (int d = 0; d < D; ++d) {
                    const int idx = num + index_offset + d * (num_offset / D);
                    const int64_t n = sizes[idx];
                    const int64_t chunk = n / 4;
                    for (int g = 0; g < 4; ++g) {
                        uint16_t* dst = buffer + offset + (int64_t)g * chunk;
                        uint16_t* src = params[idx] + (int64_t)perm[g] * chunk;
                        if (unpack)
                            memcpy(src, dst, sizeof(uint16_t) * (size_t)chunk);
                        else
                            memcpy(dst, src, sizeof(uint16_t) * (size_t)chunk);
                    }
                    offset += n;
                }
            }
        }
    }
}
