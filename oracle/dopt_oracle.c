/*
 * dopt_oracle.c -- CPU oracle for the dopt device-backend hot path.
 *
 * TEST INFRASTRUCTURE ONLY (see dopt_oracle.h).  Build with the Makefile beside this
 * file: -O2 -ffp-contract=off -fno-fast-math, so that every fp32 expression is rounded
 * exactly once per operator, as the reference's un-fused op graph does.
 *
 * Pinning status (which independent evidence checks each function; the tests live in
 * tests/test_oracle_*.py):
 *   ref_pointwise      IEEE closed forms via numpy float32/int32; exp/log/pow vs float64 libm
 *   ref_matmul/f64     reference KAT core/ops/math.d:212-231 + numpy float64 matmul
 *   ref_sum/max/argmin reference KATs core/ops/math.d:285-298,318-331,361-373 + numpy reductions
 *   ref_slice/pad/transpose/repeat  KATs core/ops/basic.d:212-226,246-260,307-314,336-356
 *                      + numpy slicing / np.pad / .T / np.tile
 *   ref_convolution, f64_conv_fwd   KAT core/ops/nnet.d:270-293 (pins the filter flip)
 *                      + scipy.signal.convolve2d + torch CPU conv2d on the flipped filter
 *   f64_conv_bwd_*     adjoint identities, central finite differences, torch CPU autograd
 *   ref_maxpool        KAT core/ops/nnet.d:333-352 + numpy block max
 *   f64_maxpool_grad   brute-force argmax incl. constructed ties (tie rule itself is this
 *                      build's choice: the reference holds no test for it)
 *   ref_softmax/f64    KAT core/ops/nnet.d:424-435 + scipy.special.softmax
 *   f64_softmax_grad   brute-force Jacobian
 *   f64_relu*, f64_add_bias*   closed forms via numpy
 *   f64_bn_*           torch CPU batch_norm float64 (y, running stats, autograd grads) +
 *                      the nnet/layers/batchnorm.d:158-177 scenario (running mean -> [3,4])
 *   ref_sgd/adam/amsgrad  numpy float32 one-ufunc-per-node evaluation of the same trees +
 *                      the fit-a-line scenario of online/{sgd,adam,amsgrad}.d unittests
 *   ref_image_transform  np.pad(mode="symmetric") + slicing + reversed views, every offset of a
 *                      small image enumerated (the reference holds no test for this class)
 */
#include "dopt_oracle.h"

#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------ */
/* pointwise (cpu/math.d:312-437)                                                        */
/* ------------------------------------------------------------------------------------ */

/* std.algorithm.comparison.max/min as used by cpu/math.d:316 (binfunc) */
static float maxf_d(float a, float b) { return a < b ? b : a; }
static float minf_d(float a, float b) { return a < b ? a : b; }
static int maxi_d(int a, int b) { return a < b ? b : a; }
static int mini_d(int a, int b) { return a < b ? a : b; }

/* std.math.pow(int, int): exponentiation by squaring, wrapping arithmetic. */
static int powi_d(int x, int n)
{
    if (n < 0) {
        if (x == 1) return 1;
        if (x == -1) return (n & 1) ? -1 : 1;
        return 0; /* the reference divides by zero for x == 0; callers avoid it */
    }
    unsigned int p = 1, v = (unsigned int)x;
    unsigned int m = (unsigned int)n;
    switch (m) {
    case 0: return 1;
    case 1: return x;
    case 2: return (int)(v * v);
    default: break;
    }
    for (;;) {
        if (m & 1) p *= v;
        m >>= 1;
        if (!m) break;
        v *= v;
    }
    return (int)p;
}

static int wrap_add(int a, int b) { return (int)((unsigned)a + (unsigned)b); }
static int wrap_sub(int a, int b) { return (int)((unsigned)a - (unsigned)b); }
static int wrap_mul(int a, int b) { return (int)((unsigned)a * (unsigned)b); }

typedef float (*unary_f)(float);
static float u_neg(float x) { return -x; }
static float u_abs(float x) { return fabsf(x); }
static float u_sgn(float x) { return (float)((x > 0) - (x < 0)); }

static unary_f find_unary(const char *op)
{
    static const struct { const char *n; unary_f f; } tab[] = {
        {"neg", u_neg}, {"abs", u_abs}, {"sgn", u_sgn}, {"exp", expf}, {"log", logf},
        {"sqrt", sqrtf}, {"sin", sinf}, {"cos", cosf}, {"tan", tanf}, {"asin", asinf},
        {"acos", acosf}, {"atan", atanf}, {"sinh", sinhf}, {"cosh", coshf}, {"tanh", tanhf},
        {"asinh", asinhf}, {"acosh", acoshf}, {"atanh", atanhf}};
    for (size_t i = 0; i < sizeof(tab) / sizeof(tab[0]); i++)
        if (!strcmp(tab[i].n, op)) return tab[i].f;
    return NULL;
}

int ref_pointwise(const char *op, int dtype, size_t n, const void *pa, const void *pb, void *pout)
{
    unary_f uf = find_unary(op);
    if (dtype == ORACLE_F32) {
        const float *a = (const float *)pa, *b = (const float *)pb;
        float *o = (float *)pout;
        if (uf) {
            for (size_t i = 0; i < n; i++) o[i] = uf(a[i]);
            return 0;
        }
#define BIN_F(name, expr) \
        if (!strcmp(op, name)) { for (size_t i = 0; i < n; i++) o[i] = (float)(expr); return 0; }
        BIN_F("add", a[i] + b[i])
        BIN_F("sub", a[i] - b[i])
        BIN_F("mul", a[i] * b[i])
        BIN_F("div", a[i] / b[i])
        BIN_F("lt", a[i] < b[i])
        BIN_F("lte", a[i] <= b[i])
        BIN_F("gt", a[i] > b[i])
        BIN_F("gte", a[i] >= b[i])
        BIN_F("eq", a[i] == b[i])
        BIN_F("neq", a[i] != b[i])
        BIN_F("max", maxf_d(a[i], b[i]))
        BIN_F("min", minf_d(a[i], b[i]))
        BIN_F("pow", powf(a[i], b[i]))
        BIN_F("atan2", atan2f(a[i], b[i]))
#undef BIN_F
        return 1;
    }
    if (dtype == ORACLE_I32) {
        const int *a = (const int *)pa, *b = (const int *)pb;
        int *o = (int *)pout;
        if (uf) {
            /* neg keeps integer arithmetic (opsymbol "-"); every other unary op casts the
               argument to float, applies the float function and casts back (cpu/math.d:418). */
            if (!strcmp(op, "neg")) {
                for (size_t i = 0; i < n; i++) o[i] = wrap_sub(0, a[i]);
            } else {
                for (size_t i = 0; i < n; i++) o[i] = (int)uf((float)a[i]);
            }
            return 0;
        }
#define BIN_I(name, expr) \
        if (!strcmp(op, name)) { for (size_t i = 0; i < n; i++) o[i] = (int)(expr); return 0; }
        BIN_I("add", wrap_add(a[i], b[i]))
        BIN_I("sub", wrap_sub(a[i], b[i]))
        BIN_I("mul", wrap_mul(a[i], b[i]))
        BIN_I("div", a[i] / b[i])
        BIN_I("lt", a[i] < b[i])
        BIN_I("lte", a[i] <= b[i])
        BIN_I("gt", a[i] > b[i])
        BIN_I("gte", a[i] >= b[i])
        BIN_I("eq", a[i] == b[i])
        BIN_I("neq", a[i] != b[i])
        BIN_I("max", maxi_d(a[i], b[i]))
        BIN_I("min", mini_d(a[i], b[i]))
        BIN_I("pow", powi_d(a[i], b[i]))
        BIN_I("atan2", atan2f((float)a[i], (float)b[i]))
#undef BIN_I
        return 1;
    }
    return 2;
}

/* ------------------------------------------------------------------------------------ */
/* matmul (cpu/math.d:70-88)                                                             */
/* ------------------------------------------------------------------------------------ */

int ref_matmul(size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    /* netlib SGEMM 'N','N' on the column-major view C^T = B^T A^T: for each column j of
       C^T (row of C), for each l, axpy over i.  beta = 0 clears first. */
    for (size_t r = 0; r < M; r++) {
        float *c = C + r * N;
        for (size_t j = 0; j < N; j++) c[j] = 0.0f;
        for (size_t l = 0; l < K; l++) {
            float t = A[r * K + l];
            const float *b = B + l * N;
            for (size_t j = 0; j < N; j++) c[j] += t * b[j];
        }
    }
    return 0;
}

int f64_matmul(size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    double *acc = (double *)malloc(sizeof(double) * (N ? N : 1));
    if (!acc) return 3;
    for (size_t r = 0; r < M; r++) {
        for (size_t j = 0; j < N; j++) acc[j] = 0.0;
        for (size_t l = 0; l < K; l++) {
            double t = A[r * K + l];
            const float *b = B + l * N;
            for (size_t j = 0; j < N; j++) acc[j] += t * (double)b[j];
        }
        for (size_t j = 0; j < N; j++) C[r * N + j] = (float)acc[j];
    }
    free(acc);
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* reductions (cpu/math.d:90-310)                                                        */
/* ------------------------------------------------------------------------------------ */

static size_t vol_of(const size_t *shape, int from, int to)
{
    size_t v = 1;
    for (int i = from; i < to; i++) v *= shape[i];
    return v;
}

/* Threads for the loops the reference hands to std.parallelism (`foreach(...; ....parallel)`: sum and maxElement over
   the outer index, cpu/math.d:102,179; repeat over its blocks, cpu/basic.d:166).  Each output element is still
   computed by one thread in the serial order, so results do not depend on the count.  1 unless the CPU-baseline
   timing asks for more. */
static int g_threads = 1;
void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int oracle_get_threads(void) { return g_threads; }

#define DEFINE_REDUCE(NAME, T, INIT, COMBINE)                                                  \
    static int NAME(const size_t *shape0, int rank, const size_t *axes, int naxes,             \
                    const T *in, T *out)                                                       \
    {                                                                                          \
        size_t shape[16];                                                                      \
        if (rank > 16) return 4;                                                               \
        for (int i = 0; i < rank; i++) shape[i] = shape0[i];                                   \
        const T *inbuf = in;                                                                   \
        T *owned_in = NULL, *outbuf = NULL;                                                    \
        size_t newvol = vol_of(shape, 0, rank);                                                \
        for (int ai = 0; ai < naxes; ai++) {                                                   \
            size_t axis = axes[ai];                                                            \
            if (axis >= (size_t)rank) { free(owned_in); return 5; }                            \
            newvol = vol_of(shape, 0, rank) / shape[axis];                                     \
            size_t lowstride = (axis == (size_t)rank - 1) ? 1 : vol_of(shape, (int)axis + 1, rank); \
            size_t highstride = lowstride * shape[axis];                                       \
            outbuf = (T *)malloc(sizeof(T) * (newvol ? newvol : 1));                           \
            if (!outbuf) { free(owned_in); return 3; }                                         \
            _Pragma("omp parallel for schedule(static) if (g_threads > 1) num_threads(g_threads)") \
            for (size_t o = 0; o < newvol / lowstride; o++) {                                  \
                if (lowstride == 1) {                                                          \
                    T acc = INIT;                                                              \
                    for (size_t i = 0; i < highstride; i++) {                                  \
                        T x = inbuf[o * highstride + i];                                       \
                        acc = COMBINE(acc, x);                                                 \
                    }                                                                          \
                    outbuf[o] = acc;                                                           \
                } else {                                                                       \
                    for (size_t j = 0; j < lowstride; j++) outbuf[o * lowstride + j] = INIT;   \
                    for (size_t i = 0; i < highstride / lowstride; i++)                        \
                        for (size_t j = 0; j < lowstride; j++) {                               \
                            T x = inbuf[o * highstride + i * lowstride + j];                   \
                            T acc = outbuf[o * lowstride + j];                                 \
                            outbuf[o * lowstride + j] = COMBINE(acc, x);                       \
                        }                                                                      \
                }                                                                              \
            }                                                                                  \
            free(owned_in);                                                                    \
            owned_in = outbuf;                                                                 \
            inbuf = outbuf;                                                                    \
            shape[axis] = 1;                                                                   \
        }                                                                                      \
        if (!outbuf) return 6; /* the reference copies a null slice here: no axes is illegal */ \
        memcpy(out, outbuf, sizeof(T) * newvol);                                               \
        free(outbuf);                                                                          \
        return 0;                                                                              \
    }

#define ADD_F(a, b) ((a) + (b))
#define ADD_I(a, b) wrap_add((a), (b))
#define MAX_F(a, b) maxf_d((a), (b))
#define MAX_I(a, b) maxi_d((a), (b))
DEFINE_REDUCE(sum_f32, float, 0.0f, ADD_F)
DEFINE_REDUCE(sum_i32, int, 0, ADD_I)
DEFINE_REDUCE(max_f32, float, -FLT_MAX, MAX_F)
DEFINE_REDUCE(max_i32, int, -INT_MAX, MAX_I)

int ref_sum(int dtype, const size_t *shape, int rank, const size_t *axes, int naxes,
            const void *in, void *out)
{
    if (dtype == ORACLE_F32) return sum_f32(shape, rank, axes, naxes, (const float *)in, (float *)out);
    if (dtype == ORACLE_I32) return sum_i32(shape, rank, axes, naxes, (const int *)in, (int *)out);
    return 2;
}

int ref_max_element(int dtype, const size_t *shape, int rank, const size_t *axes, int naxes,
                    const void *in, void *out)
{
    if (dtype == ORACLE_F32) return max_f32(shape, rank, axes, naxes, (const float *)in, (float *)out);
    if (dtype == ORACLE_I32) return max_i32(shape, rank, axes, naxes, (const int *)in, (int *)out);
    return 2;
}

int ref_argmin(int dtype, const size_t *shape, int rank, size_t axis, const void *in, int32_t *out)
{
    if (axis >= (size_t)rank) return 5;
    size_t outer = vol_of(shape, 0, (int)axis);
    size_t inner = shape[axis];
    size_t vol = vol_of(shape, (int)axis + 1, rank);
    if (dtype == ORACLE_F32) {
        const float *inbuf = (const float *)in;
        float *vals = (float *)malloc(sizeof(float) * (vol ? vol : 1));
        if (!vals) return 3;
        for (size_t o = 0; o < outer; o++) {
            for (size_t j = 0; j < vol; j++) vals[j] = FLT_MAX;
            for (size_t i = 0; i < inner; i++)
                for (size_t j = 0; j < vol; j++)
                    if (inbuf[o * vol * inner + i * vol + j] < vals[j]) {
                        vals[j] = inbuf[o * vol * inner + i * vol + j];
                        out[o * vol + j] = (int32_t)i;
                    }
        }
        free(vals);
        return 0;
    }
    if (dtype == ORACLE_I32) {
        const int *inbuf = (const int *)in;
        int *vals = (int *)malloc(sizeof(int) * (vol ? vol : 1));
        if (!vals) return 3;
        for (size_t o = 0; o < outer; o++) {
            for (size_t j = 0; j < vol; j++) vals[j] = INT_MAX;
            for (size_t i = 0; i < inner; i++)
                for (size_t j = 0; j < vol; j++)
                    if (inbuf[o * vol * inner + i * vol + j] < vals[j]) {
                        vals[j] = inbuf[o * vol * inner + i * vol + j];
                        out[o * vol + j] = (int32_t)i;
                    }
        }
        free(vals);
        return 0;
    }
    return 2;
}

/* ------------------------------------------------------------------------------------ */
/* layout ops (cpu/basic.d) -- element size is hard-coded to 4 bytes there (basic.d:23,68) */
/* ------------------------------------------------------------------------------------ */

static void slice_impl(const unsigned char *in, const size_t *inShape, int rank, size_t inVol,
                       unsigned char *out, const size_t *outShape, size_t outVol,
                       const size_t *offset)
{
    const size_t size = 4;
    if (rank == 0) {
        memcpy(out, in, size);
    } else if (rank == 1) {
        memcpy(out, in + offset[0] * size, outShape[0] * size);
    } else {
        for (size_t i = 0; i < outShape[0]; i++)
            slice_impl(in + (i + offset[0]) * inVol * size, inShape + 1, rank - 1, inVol / inShape[1],
                       out + i * outVol * size, outShape + 1, outVol / outShape[1], offset + 1);
    }
}

int ref_slice(int rank, const size_t *inShape, const size_t *outShape, const size_t *start,
              const void *in, void *out)
{
    size_t inVol = vol_of(inShape, 0, rank), outVol = vol_of(outShape, 0, rank);
    if (rank > 0) { inVol /= inShape[0]; outVol /= outShape[0]; }
    slice_impl((const unsigned char *)in, inShape, rank, inVol, (unsigned char *)out, outShape, outVol, start);
    return 0;
}

static void pad_impl(const unsigned char *in, const size_t *inShape, int rank, size_t inVol,
                     unsigned char *out, size_t outBytes, const size_t *outShape, size_t outVol,
                     const size_t *offset)
{
    const size_t size = 4;
    if (rank == 0) {
        memcpy(out, in, size);
    } else if (rank == 1) {
        memset(out, 0, offset[0] * size);
        memcpy(out + offset[0] * size, in, inShape[0] * size);
        memset(out + (offset[0] + inShape[0]) * size, 0, outBytes - (offset[0] + inShape[0]) * size);
    } else {
        memset(out, 0, offset[0] * outVol * size);
        for (size_t i = 0; i < inShape[0]; i++)
            pad_impl(in + i * inVol * size, inShape + 1, rank - 1, inVol / inShape[1],
                     out + (i + offset[0]) * outVol * size, outVol * size, outShape + 1,
                     outVol / outShape[1], offset + 1);
        memset(out + (offset[0] + inShape[0]) * outVol * size, 0,
               outBytes - (offset[0] + inShape[0]) * outVol * size);
    }
}

int ref_pad(int rank, const size_t *inShape, const size_t *outShape, const size_t *before,
            const void *in, void *out)
{
    size_t inVol = vol_of(inShape, 0, rank), outVol = vol_of(outShape, 0, rank);
    size_t outBytes = outVol * 4;
    if (rank > 0) { inVol /= inShape[0]; outVol /= outShape[0]; }
    pad_impl((const unsigned char *)in, inShape, rank, inVol, (unsigned char *)out, outBytes, outShape, outVol, before);
    return 0;
}

int ref_transpose(size_t inRows, size_t inCols, const void *in, void *out)
{
    /* cpu/basic.d:137-151 with rows/cols of the OUTPUT: out[r][c] = in[c][r]. */
    const uint32_t *src = (const uint32_t *)in;
    uint32_t *dst = (uint32_t *)out;
    size_t rows = inCols, cols = inRows;
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < cols; c++) dst[r * cols + c] = src[c * rows + r];
    return 0;
}

int ref_repeat(int rank, const size_t *inShape, const size_t *reps, const void *in, void *out)
{
    /* cpu/basic.d:155-205: one pass per axis, innermost first; blocks of `vol` elements are
       each written `reps` times back to back. */
    size_t vol = 1;
    size_t len = vol_of(inShape, 0, rank);
    const uint32_t *inbuf = (const uint32_t *)in;
    uint32_t *owned = NULL, *outbuf = NULL;
    for (int ax = rank - 1; ax >= 0; ax--) {
        size_t a = reps[ax];
        vol *= inShape[ax];
        outbuf = (uint32_t *)malloc(4 * ((len * a) != 0 ? len * a : 1));
        if (!outbuf) { free(owned); return 3; }
        /* cpu/basic.d:166: the blocks are handed to the task pool */
#pragma omp parallel for schedule(static) if (g_threads > 1) num_threads(g_threads)
        for (size_t b = 0; b < len / vol; b++) {
            const size_t i = b * vol;
            for (size_t o = i * a; o < (i + vol) * a; o += vol) memcpy(outbuf + o, inbuf + i, vol * 4);
        }
        vol *= a;
        len *= a;
        free(owned);
        owned = outbuf;
        inbuf = outbuf;
    }
    if (!outbuf) { /* rank 0: the reference copies a null slice; treat as identity */
        memcpy(out, in, 4);
        return 0;
    }
    memcpy(out, outbuf, len * 4);
    free(outbuf);
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* convolution                                                                           */
/* ------------------------------------------------------------------------------------ */

static size_t conv_out(size_t in, size_t pad, size_t k, size_t stride)
{
    return (in + 2 * pad - k) / stride + 1; /* core/ops/nnet.d:71-87 */
}

int ref_convolution(const oracle_conv_desc *d, const float *x, const float *w, float *y)
{
    size_t P = conv_out(d->H, d->padH, d->R, d->strideH), Q = conv_out(d->W, d->padW, d->S, d->strideW);
    size_t inVol = d->H * d->W, outVol = P * Q, kernVol = d->R * d->S;
    for (size_t b = 0; b < d->N; b++)
        for (size_t o = 0; o < d->K; o++) {
            float *outimg = y + (b * d->K + o) * outVol;
            for (size_t i = 0; i < outVol; i++) outimg[i] = 0.0f;
            for (size_t c = 0; c < d->C; c++) {
                const float *inimg = x + (b * d->C + c) * inVol;
                const float *kern = w + (o * d->C + c) * kernVol;
                size_t outidx = 0;
                for (size_t yy = 0; yy < P; yy++)
                    for (size_t xx = 0; xx < Q; xx++) {
                        float outval = 0.0f;
                        for (size_t j = 0; j < d->R; j++) {
                            size_t jprime = d->R - j - 1;
                            for (size_t i = 0; i < d->S; i++) {
                                size_t iprime = d->S - i - 1;
                                ptrdiff_t iny = (ptrdiff_t)(yy * d->strideH) - (ptrdiff_t)d->padH + (ptrdiff_t)j;
                                ptrdiff_t inx = (ptrdiff_t)(xx * d->strideW) - (ptrdiff_t)d->padW + (ptrdiff_t)i;
                                /* cpu/nnet.d:54 tests against the OUTPUT dims */
                                if (0 <= iny && iny < (ptrdiff_t)P && 0 <= inx && inx < (ptrdiff_t)Q)
                                    outval += kern[jprime * d->S + iprime] * inimg[iny * (ptrdiff_t)d->W + inx];
                            }
                        }
                        outimg[outidx] += outval;
                        outidx++;
                    }
            }
        }
    return 0;
}

int f64_conv_fwd(const oracle_conv_desc *d, const float *x, const float *w, float *y)
{
    size_t P = conv_out(d->H, d->padH, d->R, d->strideH), Q = conv_out(d->W, d->padW, d->S, d->strideW);
    for (size_t n = 0; n < d->N; n++)
        for (size_t k = 0; k < d->K; k++)
            for (size_t p = 0; p < P; p++)
                for (size_t q = 0; q < Q; q++) {
                    double acc = 0.0;
                    for (size_t c = 0; c < d->C; c++)
                        for (size_t r = 0; r < d->R; r++)
                            for (size_t s = 0; s < d->S; s++) {
                                ptrdiff_t ih = (ptrdiff_t)(p * d->strideH + r) - (ptrdiff_t)d->padH;
                                ptrdiff_t iw = (ptrdiff_t)(q * d->strideW + s) - (ptrdiff_t)d->padW;
                                if (ih < 0 || iw < 0 || ih >= (ptrdiff_t)d->H || iw >= (ptrdiff_t)d->W) continue;
                                acc += (double)x[((n * d->C + c) * d->H + (size_t)ih) * d->W + (size_t)iw] *
                                       (double)w[((k * d->C + c) * d->R + (d->R - 1 - r)) * d->S + (d->S - 1 - s)];
                            }
                    y[((n * d->K + k) * P + p) * Q + q] = (float)acc;
                }
    return 0;
}

int f64_conv_bwd_data(const oracle_conv_desc *d, const float *dy, const float *w, float *dx)
{
    size_t P = conv_out(d->H, d->padH, d->R, d->strideH), Q = conv_out(d->W, d->padW, d->S, d->strideW);
    size_t nx = d->N * d->C * d->H * d->W;
    double *acc = (double *)calloc(nx ? nx : 1, sizeof(double));
    if (!acc) return 3;
    for (size_t n = 0; n < d->N; n++)
        for (size_t k = 0; k < d->K; k++)
            for (size_t p = 0; p < P; p++)
                for (size_t q = 0; q < Q; q++) {
                    double g = dy[((n * d->K + k) * P + p) * Q + q];
                    for (size_t c = 0; c < d->C; c++)
                        for (size_t r = 0; r < d->R; r++)
                            for (size_t s = 0; s < d->S; s++) {
                                ptrdiff_t ih = (ptrdiff_t)(p * d->strideH + r) - (ptrdiff_t)d->padH;
                                ptrdiff_t iw = (ptrdiff_t)(q * d->strideW + s) - (ptrdiff_t)d->padW;
                                if (ih < 0 || iw < 0 || ih >= (ptrdiff_t)d->H || iw >= (ptrdiff_t)d->W) continue;
                                acc[((n * d->C + c) * d->H + (size_t)ih) * d->W + (size_t)iw] +=
                                    g * (double)w[((k * d->C + c) * d->R + (d->R - 1 - r)) * d->S + (d->S - 1 - s)];
                            }
                }
    for (size_t i = 0; i < nx; i++) dx[i] = (float)acc[i];
    free(acc);
    return 0;
}

int f64_conv_bwd_filter(const oracle_conv_desc *d, const float *dy, const float *x, float *dw)
{
    size_t P = conv_out(d->H, d->padH, d->R, d->strideH), Q = conv_out(d->W, d->padW, d->S, d->strideW);
    size_t nw = d->K * d->C * d->R * d->S;
    double *acc = (double *)calloc(nw ? nw : 1, sizeof(double));
    if (!acc) return 3;
    for (size_t n = 0; n < d->N; n++)
        for (size_t k = 0; k < d->K; k++)
            for (size_t p = 0; p < P; p++)
                for (size_t q = 0; q < Q; q++) {
                    double g = dy[((n * d->K + k) * P + p) * Q + q];
                    for (size_t c = 0; c < d->C; c++)
                        for (size_t r = 0; r < d->R; r++)
                            for (size_t s = 0; s < d->S; s++) {
                                ptrdiff_t ih = (ptrdiff_t)(p * d->strideH + r) - (ptrdiff_t)d->padH;
                                ptrdiff_t iw = (ptrdiff_t)(q * d->strideW + s) - (ptrdiff_t)d->padW;
                                if (ih < 0 || iw < 0 || ih >= (ptrdiff_t)d->H || iw >= (ptrdiff_t)d->W) continue;
                                acc[((k * d->C + c) * d->R + (d->R - 1 - r)) * d->S + (d->S - 1 - s)] +=
                                    g * (double)x[((n * d->C + c) * d->H + (size_t)ih) * d->W + (size_t)iw];
                            }
                }
    for (size_t i = 0; i < nw; i++) dw[i] = (float)acc[i];
    free(acc);
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* pooling / softmax                                                                     */
/* ------------------------------------------------------------------------------------ */

int ref_maxpool(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw, const float *x, float *y)
{
    size_t P = H / ph, Q = W / pw; /* core/ops/nnet.d:97-107 */
    for (size_t m = 0; m < N * C; m++) {
        const float *inimg = x + m * H * W;
        float *outimg = y + m * P * Q;
        for (size_t yy = 0; yy < P; yy++)
            for (size_t xx = 0; xx < Q; xx++) {
                float maxval = -FLT_MAX;
                for (size_t j = 0; j < ph; j++)
                    for (size_t i = 0; i < pw; i++)
                        maxval = maxf_d(maxval, inimg[(yy * ph + j) * W + xx * pw + i]);
                outimg[yy * Q + xx] = maxval;
            }
    }
    return 0;
}

int f64_maxpool_grad(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw,
                     const float *dy, const float *x, float *dx)
{
    size_t P = H / ph, Q = W / pw;
    memset(dx, 0, sizeof(float) * N * C * H * W);
    for (size_t m = 0; m < N * C; m++) {
        const float *inimg = x + m * H * W;
        float *gimg = dx + m * H * W;
        for (size_t yy = 0; yy < P; yy++)
            for (size_t xx = 0; xx < Q; xx++) {
                /* the element the forward loop (cpu/nnet.d:103-113: acc = max(acc, v) = acc < v ? v : acc from
                   -float.max) ends up holding: first maximum in row-major order, a NaN never; the window's first
                   element when no test fires */
                size_t best = (yy * ph) * W + xx * pw;
                float bestv = -FLT_MAX;
                for (size_t j = 0; j < ph; j++)
                    for (size_t i = 0; i < pw; i++) {
                        size_t idx = (yy * ph + j) * W + xx * pw + i;
                        if (bestv < inimg[idx]) { bestv = inimg[idx]; best = idx; }
                    }
                gimg[best] = dy[m * P * Q + yy * Q + xx];
            }
    }
    return 0;
}

int ref_softmax(size_t N, size_t C, size_t inner, const float *x, float *y)
{
    for (size_t b = 0; b < N; b++)
        for (size_t i = 0; i < inner; i++) {
            float m = -FLT_MAX;
            for (size_t o = 0; o < C; o++) m = maxf_d(m, x[b * C * inner + o * inner + i]);
            float s = 0.0f;
            for (size_t o = 0; o < C; o++) {
                float pot = expf(x[b * C * inner + o * inner + i] - m);
                s += pot;
                y[b * C * inner + o * inner + i] = pot;
            }
            for (size_t o = 0; o < C; o++) y[b * C * inner + o * inner + i] /= s;
        }
    return 0;
}

int f64_softmax(size_t N, size_t C, size_t inner, const float *x, float *y)
{
    for (size_t b = 0; b < N; b++)
        for (size_t i = 0; i < inner; i++) {
            double m = -DBL_MAX, s = 0.0;
            for (size_t o = 0; o < C; o++) m = fmax(m, (double)x[b * C * inner + o * inner + i]);
            for (size_t o = 0; o < C; o++) s += exp((double)x[b * C * inner + o * inner + i] - m);
            for (size_t o = 0; o < C; o++)
                y[b * C * inner + o * inner + i] = (float)(exp((double)x[b * C * inner + o * inner + i] - m) / s);
        }
    return 0;
}

int f64_softmax_grad(size_t N, size_t C, size_t inner, const float *dy, const float *y, float *dx)
{
    for (size_t b = 0; b < N; b++)
        for (size_t i = 0; i < inner; i++) {
            double dot = 0.0;
            for (size_t o = 0; o < C; o++) {
                size_t idx = b * C * inner + o * inner + i;
                dot += (double)dy[idx] * (double)y[idx];
            }
            for (size_t o = 0; o < C; o++) {
                size_t idx = b * C * inner + o * inner + i;
                dx[idx] = (float)((double)y[idx] * ((double)dy[idx] - dot));
            }
        }
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* relu / bias                                                                           */
/* ------------------------------------------------------------------------------------ */

int f64_relu(size_t n, const float *x, float *y)
{
    for (size_t i = 0; i < n; i++) y[i] = x[i] < 0.0f ? 0.0f : x[i]; /* NaN propagates */
    return 0;
}

int f64_relu_grad(size_t n, const float *dy, const float *x, float *dx)
{
    for (size_t i = 0; i < n; i++) dx[i] = x[i] > 0.0f ? dy[i] : 0.0f;
    return 0;
}

int f64_add_bias(size_t N, size_t C, size_t inner, const float *x, const float *b, float *y)
{
    for (size_t n = 0; n < N; n++)
        for (size_t c = 0; c < C; c++)
            for (size_t i = 0; i < inner; i++) {
                size_t idx = (n * C + c) * inner + i;
                y[idx] = x[idx] + b[c];
            }
    return 0;
}

int f64_add_bias_grad(size_t N, size_t C, size_t inner, const float *dy, float *db)
{
    for (size_t c = 0; c < C; c++) {
        double acc = 0.0;
        for (size_t n = 0; n < N; n++)
            for (size_t i = 0; i < inner; i++) acc += (double)dy[(n * C + c) * inner + i];
        db[c] = (float)acc;
    }
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* batch normalisation (spatial mode; cudnn7.d:547-654)                                  */
/* ------------------------------------------------------------------------------------ */

static void bn_stats(size_t N, size_t C, size_t inner, size_t c, const float *x, double *mean, double *var)
{
    double m = (double)(N * inner), s = 0.0, ss = 0.0;
    for (size_t n = 0; n < N; n++)
        for (size_t i = 0; i < inner; i++) s += (double)x[(n * C + c) * inner + i];
    double mu = s / m;
    for (size_t n = 0; n < N; n++)
        for (size_t i = 0; i < inner; i++) {
            double dlt = (double)x[(n * C + c) * inner + i] - mu;
            ss += dlt * dlt;
        }
    *mean = mu;
    *var = ss / m; /* biased */
}

int f64_bn_train(size_t N, size_t C, size_t inner, double momentum, const float *x,
                 const float *scale, const float *bias, const float *runMean, const float *runVar,
                 float *packed)
{
    size_t vol = N * C * inner;
    double m = (double)(N * inner);
    double eps = (double)1e-5f;            /* cudnn7.d:610 passes the float literal */
    double factor = 1.0 - momentum;        /* cudnn7.d:592 */
    for (size_t c = 0; c < C; c++) {
        double mu, var;
        bn_stats(N, C, inner, c, x, &mu, &var);
        double rstd = 1.0 / sqrt(var + eps);
        for (size_t n = 0; n < N; n++)
            for (size_t i = 0; i < inner; i++) {
                size_t idx = (n * C + c) * inner + i;
                packed[idx] = (float)((double)scale[c] * (((double)x[idx] - mu) * rstd) + (double)bias[c]);
            }
        double unbiased = m > 1.0 ? var * m / (m - 1.0) : var;
        packed[vol + c] = (float)((1.0 - factor) * (double)runMean[c] + factor * mu);
        packed[vol + C + c] = (float)((1.0 - factor) * (double)runVar[c] + factor * unbiased);
    }
    return 0;
}

int f64_bn_grad(size_t N, size_t C, size_t inner, const float *dy, const float *x, const float *scale,
                float *packed)
{
    size_t vol = N * C * inner;
    double m = (double)(N * inner);
    double eps = (double)1e-5f; /* cudnn7.d:634 */
    for (size_t c = 0; c < C; c++) {
        double mu, var;
        bn_stats(N, C, inner, c, x, &mu, &var);
        double rstd = 1.0 / sqrt(var + eps);
        double dbias = 0.0, dscale = 0.0;
        for (size_t n = 0; n < N; n++)
            for (size_t i = 0; i < inner; i++) {
                size_t idx = (n * C + c) * inner + i;
                dbias += (double)dy[idx];
                dscale += (double)dy[idx] * (((double)x[idx] - mu) * rstd);
            }
        for (size_t n = 0; n < N; n++)
            for (size_t i = 0; i < inner; i++) {
                size_t idx = (n * C + c) * inner + i;
                double xhat = ((double)x[idx] - mu) * rstd;
                packed[idx] = (float)((double)scale[c] * rstd / m * (m * (double)dy[idx] - dbias - xhat * dscale));
            }
        packed[vol + c] = (float)dscale;
        packed[vol + C + c] = (float)dbias;
    }
    return 0;
}

int f64_bn_infer(size_t N, size_t C, size_t inner, const float *x, const float *scale,
                 const float *bias, const float *mean, const float *var, float *y)
{
    double eps = 1e-5; /* cudnn7.d:652 passes the double literal */
    for (size_t n = 0; n < N; n++)
        for (size_t c = 0; c < C; c++) {
            double rstd = 1.0 / sqrt((double)var[c] + eps);
            for (size_t i = 0; i < inner; i++) {
                size_t idx = (n * C + c) * inner + i;
                y[idx] = (float)((double)scale[c] * (((double)x[idx] - (double)mean[c]) * rstd) + (double)bias[c]);
            }
        }
    return 0;
}

/* ------------------------------------------------------------------------------------ */
/* optimizers: every node of the reference expression tree is its own fp32 rounding       */
/* ------------------------------------------------------------------------------------ */

int ref_sgd_step(size_t n, float lr, float mu, int nesterov, const float *w, const float *g,
                 const float *mom, float *wOut, float *momOut)
{
    for (size_t i = 0; i < n; i++) {
        volatile float a = mom[i] * mu;  /* x[1] * momentumRate      (sgd.d:48,59) */
        volatile float b = lr * g[i];    /* learningRate * x[0]                   */
        if (nesterov) {
            volatile float nm = a - b;                 /* sgd.d:48 */
            volatile float t0 = mu * nm;               /* momentumRate * x[1]   (sgd.d:52) */
            volatile float t1 = w[i] + t0;
            volatile float t2 = lr * g[i];
            momOut[i] = nm;
            wOut[i] = t1 - t2;
        } else {
            volatile float nm = a + b;                 /* sgd.d:59 */
            momOut[i] = nm;
            wOut[i] = w[i] - nm;                       /* sgd.d:63 */
        }
    }
    return 0;
}

int ref_adam_scalars(float alpha, float beta1, float beta2, float b1, float b2,
                     float *nb1, float *nb2, float *eta)
{
    volatile float n1 = b1 * beta1;          /* adam.d:48 */
    volatile float n2 = b2 * beta2;          /* adam.d:49 */
    volatile float one_m_n2 = 1.0f - n2;
    volatile float sq = sqrtf(one_m_n2);
    volatile float num = alpha * sq;
    volatile float den = 1.0f - n1;
    *nb1 = n1;
    *nb2 = n2;
    *eta = num / den;                        /* adam.d:50: (alpha * sqrt(1 - nb2)) / (1 - nb1) */
    return 0;
}

int ref_adam_step(size_t n, float eta, float beta1, float beta2, float eps, const float *w,
                  const float *g, const float *m, const float *v, float *wOut, float *mOut, float *vOut)
{
    volatile float c1 = 1.0f - beta1, c2 = 1.0f - beta2;
    for (size_t i = 0; i < n; i++) {
        volatile float t0 = beta1 * m[i];
        volatile float t1 = c1 * g[i];
        volatile float nm = t0 + t1;         /* adam.d:54 */
        volatile float t2 = beta2 * v[i];
        volatile float t3 = c2 * g[i];
        volatile float t4 = t3 * g[i];       /* ((1 - beta2) * g) * g */
        volatile float nv = t2 + t4;         /* adam.d:59 */
        volatile float sq = sqrtf(nv);
        volatile float den = sq + eps;
        volatile float q = nm / den;
        volatile float step = eta * q;
        mOut[i] = nm;
        vOut[i] = nv;
        wOut[i] = w[i] - step;               /* adam.d:63 */
    }
    return 0;
}

int ref_amsgrad_step(size_t n, float eta, float beta1, float beta2, float eps, const float *w,
                     const float *g, const float *m, const float *v, const float *vhat,
                     float *wOut, float *mOut, float *vOut, float *vhatOut)
{
    /* vhat' = max(vhat, OLD v) is computed before v may be overwritten in place. */
    for (size_t i = 0; i < n; i++) vhatOut[i] = maxf_d(vhat[i], v[i]); /* amsgrad.d:63-66 */
    return ref_adam_step(n, eta, beta1, beta2, eps, w, g, m, v, wOut, mOut, vOut);
}

/* ---- nnet/data/imagetransformer.d:45-138 (ImageTransformer.getBatch), one image at a time ----
 * The loops, the padded scratch image and the in-place reversals are the reference's; the random
 * draws (xOff, yOff, the two coin flips) are arguments here.  `img` is transformed in place, as in
 * the reference; `padded` holds C * (H + 2 jy) * (W + 2 jx) floats. */
static void reverse_run(float *a, size_t n, size_t stride)
{
    for (size_t i = 0; i < n / 2; i++) {
        float t = a[i * stride];
        a[i * stride] = a[(n - 1 - i) * stride];
        a[(n - 1 - i) * stride] = t;
    }
}

int ref_image_transform(size_t N, size_t C, size_t H, size_t W, size_t jx, size_t jy,
                        const int32_t *geom, float *batch, float *padded)
{
    const size_t pw = W + 2 * jx, ph = H + 2 * jy;
    for (size_t n = 0; n < N; n++) {
        float *img = batch + n * C * H * W;
        const size_t xOff = (size_t)geom[3 * n], yOff = (size_t)geom[3 * n + 1];
        const int flipX = geom[3 * n + 2] & 1, flipY = geom[3 * n + 2] & 2;
        if (jx != 0 || jy != 0) {                                    /* :58 */
            for (size_t c = 0; c < C; c++) {
                for (size_t y = 0; y < H; y++) {
                    for (size_t x = 0; x < W; x++)                   /* :65-69 */
                        padded[c * ph * pw + (y + jy) * pw + x + jx] = img[c * H * W + y * W + x];
                    if (jx != 0) {                                   /* :71-80 */
                        size_t o = c * ph * pw + (y + jy) * pw;
                        memcpy(padded + o, padded + o + jx, jx * sizeof(float));
                        reverse_run(padded + o, jx, 1);
                        o += W;
                        memcpy(padded + o + jx, padded + o, jx * sizeof(float));
                        reverse_run(padded + o + jx, jx, 1);
                    }
                }
                for (size_t y = 0; y < jy; y++) {                    /* :83-94 */
                    const size_t o = c * pw * ph;
                    memcpy(padded + o + y * pw, padded + o + (2 * jy - y - 1) * pw, pw * sizeof(float));
                    memcpy(padded + o + (ph - y - 1) * pw, padded + o + (ph - 2 * jy + y) * pw, pw * sizeof(float));
                }
            }
            for (size_t c = 0; c < C; c++)                           /* :100-110 */
                for (size_t y = 0; y < H; y++)
                    for (size_t x = 0; x < W; x++)
                        img[c * H * W + y * W + x] = padded[c * ph * pw + (y + yOff) * pw + x + xOff];
        }
        if (flipX)                                                   /* :113-119: every row of every channel */
            for (size_t r = 0; r < C * H; r++) reverse_run(img + r * W, W, 1);
        if (flipY)                                                   /* :121-132: every column of every channel */
            for (size_t c = 0; c < C; c++)
                for (size_t x = 0; x < W; x++) reverse_run(img + c * H * W + x, H, W);
    }
    return 0;
}
