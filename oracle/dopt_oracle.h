/*
 * dopt_oracle.h -- CPU oracle for the dopt device-backend hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls
 * this code; it exists so that the HIP kernels can be checked against a CPU
 * restatement of what the reference computes.
 *
 * Two families of functions live here:
 *
 *  ref_*   float32 restatements of the reference CPU evaluator, loop for loop
 *          (cpu/source/dopt/cpu/{math,basic,nnet}.d) and of the optimizer expression
 *          trees (online/source/dopt/online/{sgd,adam,amsgrad}.d), every node rounded
 *          separately in fp32 exactly as the un-fused reference graph does.
 *
 *  f64_*   float64 direct-loop definitions of the operations that only cuDNN
 *          implements in the reference (cuda/source/dopt/cuda/nnet/cudnn7.d), written to
 *          the reference's own op semantics (true convolution: the filter is flipped).
 *          Inputs/outputs are float32, accumulation is float64, one final rounding.
 *
 * All pointers are host pointers, tensors are dense row-major, sizes are element
 * counts.  Every function returns 0 on success and a non-zero code for an argument it
 * refuses (the reference throws in those places).
 */
#ifndef DOPT_ORACLE_H
#define DOPT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORACLE_F32 = 0, ORACLE_I32 = 1 };

/* cpu/math.d:312-437 -- generated pointwise kernels. `op` is the reference op name. */
int ref_pointwise(const char *op, int dtype, size_t n, const void *a, const void *b, void *out);

/* cpu/math.d:70-88 -- row-major C[M,N] = A[M,K] * B[K,N], fp32 accumulation in the
   netlib reference-BLAS loop order (the reference calls system BLAS). */
int ref_matmul(size_t M, size_t N, size_t K, const float *A, const float *B, float *C);
/* float64-accumulated definition of the same product. */
int f64_matmul(size_t M, size_t N, size_t K, const float *A, const float *B, float *C);

/* cpu/math.d:90-168, 170-247 -- axis-at-a-time reductions. */
int ref_sum(int dtype, const size_t *shape, int rank, const size_t *axes, int naxes,
            const void *in, void *out);
int ref_max_element(int dtype, const size_t *shape, int rank, const size_t *axes, int naxes,
                    const void *in, void *out);
/* cpu/math.d:249-310 -- `out` (int32) must arrive zero-filled like a fresh output buffer. */
int ref_argmin(int dtype, const size_t *shape, int rank, size_t axis, const void *in, int32_t *out);

/* cpu/basic.d:21-64, 66-115, 117-153, 155-205 */
int ref_slice(int rank, const size_t *inShape, const size_t *outShape, const size_t *start,
              const void *in, void *out);
int ref_pad(int rank, const size_t *inShape, const size_t *outShape, const size_t *before,
            const void *in, void *out);
int ref_transpose(size_t inRows, size_t inCols, const void *in, void *out);
int ref_repeat(int rank, const size_t *inShape, const size_t *reps, const void *in, void *out);

typedef struct {
    size_t N, C, H, W;     /* features  [N,C,H,W]  */
    size_t K, R, S;        /* filters   [K,C,R,S]  */
    size_t padH, padW, strideH, strideW;
} oracle_conv_desc;

/* cpu/nnet.d:20-87 including its bounds test against the OUTPUT dims (nnet.d:54). */
int ref_convolution(const oracle_conv_desc *d, const float *x, const float *w, float *y);
/* cuda/nnet/cudnn7.d:113-249 -- CUDNN_CONVOLUTION (flipped filter) forward, data grad, filter grad. */
int f64_conv_fwd(const oracle_conv_desc *d, const float *x, const float *w, float *y);
int f64_conv_bwd_data(const oracle_conv_desc *d, const float *dy, const float *w, float *dx);
int f64_conv_bwd_filter(const oracle_conv_desc *d, const float *dy, const float *x, float *dw);

/* cpu/nnet.d:89-127 */
int ref_maxpool(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw, const float *x, float *y);
/* cudnn7.d:309-333 -- gradient routed to the first maximum of each window (row-major scan). */
int f64_maxpool_grad(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw,
                     const float *dy, const float *x, float *dx);

/* cpu/nnet.d:129-166 */
int ref_softmax(size_t N, size_t C, size_t inner, const float *x, float *y);
int f64_softmax(size_t N, size_t C, size_t inner, const float *x, float *y);
/* cudnn7.d:373-404 */
int f64_softmax_grad(size_t N, size_t C, size_t inner, const float *dy, const float *y, float *dx);

/* cudnn7.d:406-545 */
int f64_relu(size_t n, const float *x, float *y);
int f64_relu_grad(size_t n, const float *dy, const float *x, float *dx);
int f64_add_bias(size_t N, size_t C, size_t inner, const float *x, const float *b, float *y);
int f64_add_bias_grad(size_t N, size_t C, size_t inner, const float *dy, float *db);

/* cudnn7.d:547-654 -- packed outputs as the op judges define them (core/ops/nnet.d:222-235). */
int f64_bn_train(size_t N, size_t C, size_t inner, double momentum, const float *x,
                 const float *scale, const float *bias, const float *runMean, const float *runVar,
                 float *packed /* [N*C*inner + 2C] */);
int f64_bn_grad(size_t N, size_t C, size_t inner, const float *dy, const float *x, const float *scale,
                float *packed /* [N*C*inner + 2C] */);
int f64_bn_infer(size_t N, size_t C, size_t inner, const float *x, const float *scale,
                 const float *bias, const float *mean, const float *var, float *y);

/* online/sgd.d:44-63 -- un-fused expression tree, one fp32 rounding per node. */
int ref_sgd_step(size_t n, float lr, float mu, int nesterov, const float *w, const float *g,
                 const float *mom, float *wOut, float *momOut);
/* online/adam.d:44-63: scalars; b1/b2 are the persisted running products. */
int ref_adam_scalars(float alpha, float beta1, float beta2, float b1, float b2,
                     float *nb1, float *nb2, float *eta);
/* online/adam.d:52-63 */
int ref_adam_step(size_t n, float eta, float beta1, float beta2, float eps, const float *w,
                  const float *g, const float *m, const float *v, float *wOut, float *mOut, float *vOut);
/* online/amsgrad.d:52-69 -- note w' uses v', and vhat' = max(vhat, OLD v). */
int ref_amsgrad_step(size_t n, float eta, float beta1, float beta2, float eps, const float *w,
                     const float *g, const float *m, const float *v, const float *vhat,
                     float *wOut, float *mOut, float *vOut, float *vhatOut);

/* nnet/data/imagetransformer.d:45-138; geom = N x {xOff, yOff, bit 0 flip X | bit 1 flip Y}. */
int ref_image_transform(size_t N, size_t C, size_t H, size_t W, size_t jx, size_t jy,
                        const int32_t *geom, float *batch, float *padded);

/* Threads for the loops the reference runs through std.parallelism (sum, maxElement, repeat); default 1.
   Results do not depend on it. */
void oracle_set_threads(int n);
int oracle_get_threads(void);

#ifdef __cplusplus
}
#endif
#endif
