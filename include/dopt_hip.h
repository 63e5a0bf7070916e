/*
 * dopt_hip.h -- C ABI of libdopthip.so, the MI355X (gfx950) kernel library behind dopt's
 * device-backend plugin interface.
 *
 * This is the surface a `dopt.hip` D package binds with `extern(C)`: each entry point
 * replaces one device call site of the reference's CUDA backend (cited per function as
 * file:line under the reference's root).  Conventions:
 *   - every function returns 0 on success; non-zero is an error code from dopt_hip_status and
 *     dopt_hip_last_error() then holds the message the D wrapper passes to `enforce`;
 *   - all tensor pointers are DEVICE pointers unless the name says host; tensors are dense,
 *     row-major (NCHW / KCRS for images and filters); sizes count elements, not bytes;
 *   - everything is enqueued on one library-owned HIP stream and returns without waiting;
 *     dopt_hip_copy_d2h and dopt_hip_sync are the synchronisation points (the reference
 *     synchronises after nearly every launch, but callers only rely on ordering and on a
 *     device-to-host read seeing finished data);
 *   - NOT thread-safe: one host thread at a time may be inside the library (the reference's registries and
 *     plans are thread-local D globals; this library keeps one process-wide device, stream pair, workspace
 *     and kernel cache instead).  The lock inside the buffer pool only protects dopt_hip_malloc /
 *     dopt_hip_free / dopt_hip_pool_* against a garbage collector's finaliser thread releasing buffers while
 *     the owning thread allocates; everything else, including the queue an entry point enqueues on and the
 *     graph-recording state, is unguarded.
 */
#ifndef DOPT_HIP_H
#define DOPT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    DOPT_HIP_OK = 0,
    DOPT_HIP_ERR_INVALID = 1,     /* argument the reference would `enforce` against */
    DOPT_HIP_ERR_RUNTIME = 2,     /* a HIP runtime call failed */
    DOPT_HIP_ERR_UNSUPPORTED = 3, /* "Element type not supported." / unknown op name */
    DOPT_HIP_ERR_OOM = 4,         /* "CUDA memory allocation failed" analogue */
    DOPT_HIP_ERR_RTC = 5          /* run-time compilation failed (log in last_error) */
} dopt_hip_status;

/* element types of core/source/dopt/core/types.d:5-14 that the backend supports
   (cuda/package.d:511-525) */
typedef enum { DOPT_HIP_F32 = 0, DOPT_HIP_I32 = 1 } dopt_hip_dtype;

/* ---------------------------------------------------------------------------------------
 * Runtime: device, stream, pooled buffers, copies.
 * ------------------------------------------------------------------------------------- */

/* cuda/package.d:36-63 (cuInit / cuCtxCreate on device 0).  Idempotent. */
int dopt_hip_init(int device);
/* Frees the pool, the workspace, cached RTC modules and the stream. */
int dopt_hip_shutdown(void);
/* Message of the last failing call on this thread ("" if none). */
const char *dopt_hip_last_error(void);

/* CUDABuffer.create, cuda/package.d:134-156: device allocation, zero-filled.  Served from a
   size-class pool over hipMalloc instead of one cuMemAlloc + GC.collect() per buffer.
   bytes == 0 yields *ptr == NULL and success (package.d:144-147). */
int dopt_hip_malloc(void **ptr, size_t bytes);
/* CUDABuffer.destroy, cuda/package.d:161-164: returns the block to the pool. */
int dopt_hip_free(void *ptr);
/* Releases every cached (free) block back to the driver. */
int dopt_hip_pool_trim(void);
/* live = bytes handed out, cached = bytes parked in the pool, device_allocs = hipMalloc calls so far. */
int dopt_hip_pool_stats(size_t *live_bytes, size_t *cached_bytes, size_t *device_allocs);

/* cuMemsetD8 (cuda/package.d:152,245; cuda/basic.d:135) */
int dopt_hip_memset(void *dst, int byte_value, size_t bytes);
/* CUDABuffer.set(void[]) -> cuMemcpyHtoD, cuda/package.d:172-176 */
int dopt_hip_copy_h2d(void *dst, const void *host_src, size_t bytes);
/* CUDABuffer.get -> cuMemcpyDtoH, cuda/package.d:207-211.  Waits for all queued work. */
int dopt_hip_copy_d2h(void *host_dst, const void *src, size_t bytes);
/* CUDABuffer.set(DeviceBuffer) -> cuMemcpyDtoD, cuda/package.d:187-190 */
int dopt_hip_copy_d2d(void *dst, const void *src, size_t bytes);
/* Page-locked host staging for the feed path.  The reference hands pageable `float[]` batches to
   CUDABuffer.set each step (examples/cifar10.d:70-76 -> cuda/package.d:172-176, a blocking
   cuMemcpyHtoD); a batch filled into memory from dopt_hip_host_alloc can instead be queued with
   dopt_hip_copy_h2d_async, which returns at once: the copy runs in stream order before the kernels
   queued after it, and the host may refill the same staging memory after the next dopt_hip_sync
   (or keep two and alternate). */
int dopt_hip_host_alloc(void **host_ptr, size_t bytes);
int dopt_hip_host_free(void *host_ptr);
int dopt_hip_copy_h2d_async(void *dst, const void *pinned_src, size_t bytes);
/* The same upload on the library's second queue: it runs BESIDE whatever the first queue is doing (the training step
   on the previous batch) instead of behind it - the copy engine moves the bytes, no compute unit is involved.
   dopt_hip_upload_join makes everything enqueued on the first queue afterwards wait for the uploads queued so far.  The
   caller must know that nothing still running reads `dst` (dopt_hip_event_sync on an event recorded behind its last
   reader).  No counterpart in the reference, whose uploads block (cuda/package.d:172-176). */
int dopt_hip_copy_h2d_beside(void *dst, const void *pinned_src, size_t bytes);
int dopt_hip_upload_join(void);
/* n device-to-device copies, in order; copies of at most 64 KiB share kernel launches.  Stands
   for the loop of cuMemcpy calls that hands a plan's outputs to the caller's buffers
   (cuda/package.d:419-422): most of them are a few hundred bytes of batch-norm statistics. */
int dopt_hip_copy_d2d_batch(int n, void *const *dst, const void *const *src, const size_t *bytes);
/* cuCtxSynchronize (cuda/nvrtc.d:111,123; cudnn7.d:157 ...) */
int dopt_hip_sync(void);
/* The hipStream_t every entry point enqueues on (for callers that record their own events). */
void *dopt_hip_stream(void);

/* Event pairs on the library stream: the device-time replacement for the host StopWatch of
   CUDAPlan.profiler (cuda/package.d:265,410-415). */
int dopt_hip_event_create(void **event);
int dopt_hip_event_record(void *event);
int dopt_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for `stop` */
/* Blocks the host until everything enqueued before the event's last record has finished: the per-buffer wait of a feed
   loop, where the reference's blocking cuMemcpyHtoD per argument (cuda/package.d:367-401) waited for the whole device. */
int dopt_hip_event_sync(void *event);
int dopt_hip_event_destroy(void *event);

/* ---------------------------------------------------------------------------------------
 * Pointwise and reductions: hipRTC-instantiated gfx950 templates (replace the NVRTC generator,
 * cuda/nvrtc.d:29-132 and cuda/math.d:129-205).  Compiled once per (op, dtype), cached.
 * ------------------------------------------------------------------------------------- */

/* cuda/math.d:89-127 with CPU-evaluator semantics (cpu/math.d:312-437).
   Binary: add sub mul div lt lte gt gte eq neq max min pow atan2  (b != NULL)
   Unary : neg abs sgn exp log sqrt sin cos tan asin acos atan sinh cosh tanh asinh acosh atanh
           (b == NULL).  The reference's CUDA backend sends everything after sqrt to a host
           round trip (cuda/package.d:81-119); here they run on the device. */
int dopt_hip_pointwise(const char *op, int dtype, size_t n, const void *a, const void *b_or_null, void *out);
/* A DAG of pointwise nodes over n-element operands as one kernel.  The reference has no counterpart:
   it launches one generated kernel per node (cuda/math.d:129-205), its operator sugar broadcasts a
   scalar by materialising `repeat(scalar, n)` first (core/ops/package.d:94-168), and row / column
   broadcasts are products with a ones vector (core/ops/basic.d:370-381).  Operand index k < nin is
   input k, of the kind in_kind[k] says: 0 an n-element tensor; 1 a one-element tensor read at every
   position; 2 one element per row and 3 one element per column of the [n / inner, inner] view of the
   operands (`inner` is ignored when no input is of kind 2 or 3).  Index nin + j is the value of node
   j.  A node reads only inputs and earlier nodes; unary nodes ignore node_rhs.  Besides the names
   dopt_hip_pointwise accepts, nodes may be "relu" and "reluGrad" (operands dy, x).  The last node's
   value is written to `out`.  Every node is rounded to its own fp32 result exactly as the
   stand-alone kernel of that op rounds it. */
int dopt_hip_pointwise_chain(int dtype, size_t n, size_t inner, int nin, const void *const *in,
                             const unsigned char *in_kind, int nnodes, const char *const *node_op,
                             const int *node_lhs, const int *node_rhs, void *out);
/* Generates and compiles the kernel of such a chain for `arch` without loading it (no GPU needed). */
int dopt_hip_pointwise_chain_compile_only(int dtype, int nin, const unsigned char *in_kind,
                                          int nnodes, const char *const *node_op, const int *node_lhs,
                                          const int *node_rhs, const char *arch);
/* 1 or 2 for the names dopt_hip_pointwise accepts, 0 otherwise. */
int dopt_hip_pointwise_arity(const char *op);

/* Position of a name dopt_hip_pointwise accepts (and of "relu", "reluGrad") in the library's table of pointwise
   operations, or -1: the `op` of a pointwise node of dopt_hip_tiny_graph. */
int dopt_hip_pointwise_index(const char *op);

/* A run of operations on tiny fp32 tensors (at most DOPT_HIP_TINY_ELEMS elements each) as ONE launch of one workgroup,
   node after node in the order given, with a workgroup barrier in between.  The reference runs each of them as a
   kernel of its own (cuda/math.d:89-127 pointwise, cuda/package.d:81-119 the host round trip for sum / maxElement,
   cudnn7.d:470-526 softmax and its gradient, cuda/basic.d:143-217 repeat); on a few hundred values each of those lasts
   as long as the gap between two kernels.  Every node computes what its stand-alone entry point computes, in the same
   order of operations, so the results are identical to calling those one by one.
   slots: the buffers the nodes name (inputs, intermediate values and results alike; the caller owns them all).
   A node writes n elements to slots[dst] + dst_offset bytes from operands at slots[a] + a_offset, slots[b] + b_offset:
     POINTWISE     op = dopt_hip_pointwise_index(name); b = -1 for a unary operation; a_kind / b_kind: 0 the operand
                   has n elements, 1 it has one element that every result reads, 2 one element per row and 3 one per
                   column of the result seen as [n / dims[0], dims[0]] (the reference broadcasts a column or a row
                   through a product [m,1] x [1,n], core/ops/basic.d:370-381: the node `mul` of kinds 2 and 3)
     REDUCE        op = 0 sum, 1 maxElement; the operand is [dims[0], dims[1], dims[2]] and dims[1] is folded
                   (n = dims[0] * dims[2]): one run of adjacent reduced axes, as dopt_hip_reduce folds it
     SOFTMAX       the operand is [dims[0], dims[1], dims[2]] = [N, C, inner], normalised over C as dopt_hip_softmax_fwd
                   does for rows of fewer than 64 classes (or inner > 1)
     SOFTMAX_GRAD  a = dy, b = y, same layout, as dopt_hip_softmax_bwd
     REPEAT        the operand has extents dims[0..3] (leading 1s for lower ranks) and is tiled reps[0..3] times */
typedef enum { DOPT_HIP_TINY_SLOTS = 48, DOPT_HIP_TINY_NODES = 40, DOPT_HIP_TINY_ELEMS = 4096 } dopt_hip_tiny_limits;
typedef enum {
    DOPT_HIP_TINY_POINTWISE = 0,
    DOPT_HIP_TINY_REDUCE = 1,
    DOPT_HIP_TINY_SOFTMAX = 2,
    DOPT_HIP_TINY_SOFTMAX_GRAD = 3,
    DOPT_HIP_TINY_REPEAT = 4
} dopt_hip_tiny_kind;
typedef struct {
    int kind, op;
    int dst, a, b;
    int a_kind, b_kind;
    int n;
    int dst_offset, a_offset, b_offset;
    int dims[4];
    int reps[4];
} dopt_hip_tiny_node;
int dopt_hip_tiny_graph(int nslots, void *const *slots, int nnodes, const dopt_hip_tiny_node *nodes);

/* `sum` / `maxElement` (op = "sum" | "maxElement"): cpu/math.d:90-247, reached in the reference through
   the host fallback cuda/package.d:81-119.  Reduces `axes` (distinct, each < rank) of a dense
   tensor; out has the reduced axes removed (core/ops/math.d:162-175). */
int dopt_hip_reduce(const char *op, int dtype, const size_t *shape, int rank,
                    const size_t *axes, int naxes, const void *in, void *out);
/* sum(mul(x, x)) over `axes` in one pass over x - the L2 penalty of a parameter as nnet/layers build it
   (`weightDecay * sum(filters * filters)`, nnet/layers/conv.d:117; the norms of nnet/layers/conv.d:131-132, 184-187): every square is rounded to
   fp32 before it is added and the sums run in dopt_hip_reduce's order, so the value is that of the two operations
   run one after the other; the product is never stored.  fp32 only. */
int dopt_hip_reduce_squares(const size_t *shape, int rank, const size_t *axes, int naxes, const float *in, float *out);
/* `argmin`: cpu/math.d:249-310.  int32 output with the reduced axis kept as size 1
   (core/ops/math.d:185-191); the first minimum wins; a lane with no element below the
   type's maximum yields index 0. */
int dopt_hip_argmin(int dtype, const size_t *shape, int rank, size_t axis, const void *in, int32_t *out);

/* Compiles the template for (op, dtype) for `arch` (e.g. "gfx950") without loading it: lets a
   machine with no GPU check that every template builds.  op may also be "sum", "maxElement", "argmin". */
int dopt_hip_rtc_compile_only(const char *op, int dtype, const char *arch);

/* ---------------------------------------------------------------------------------------
 * Layout ops on 4-byte elements (cuda/basic.d hard-codes size = 4 at :40,:95).
 * ------------------------------------------------------------------------------------- */

/* `slice`: cuda/basic.d:31-84 (one cuMemcpy per innermost row there; one kernel here). */
int dopt_hip_slice(int rank, const size_t *in_shape, const size_t *out_shape, const size_t *start,
                   const void *in, void *out);
/* `pad`: cuda/basic.d:86-141 (memset + row copies there; one kernel writing every element here). */
int dopt_hip_pad(int rank, const size_t *in_shape, const size_t *out_shape, const size_t *before,
                 const void *in, void *out);
/* `repeat`: cuda/basic.d:143-217; tiling order pinned by core/ops/basic.d:336-356. */
int dopt_hip_repeat(int rank, const size_t *in_shape, const size_t *reps, const void *in, void *out);
/* `transpose` of a rank-2 tensor [rows, cols] -> [cols, rows]: cublasSgeam at cuda/basic.d:237-238. */
int dopt_hip_transpose2d(size_t rows, size_t cols, const void *in, void *out);

/* ---------------------------------------------------------------------------------------
 * Dense and convolution (fp32 MFMA).
 * ------------------------------------------------------------------------------------- */

/* `matmul`: cublasSgemm_v2 at cuda/math.d:234-235.  Row-major C[M,N] = A[M,K] * B[K,N],
   alpha = 1, beta = 0, no transposes.  K == 1 (broadcast outer product), N == 1 and M == 1
   (matrix-vector) take bandwidth-bound paths: the reference routes scalar broadcasts and
   row/column sums through matmul (core/ops/basic.d:370-381, core/ops/math.d:257-279). */
int dopt_hip_sgemm(size_t M, size_t N, size_t K, const float *A, const float *B, float *C);
/* The same product with either operand read transposed, as cublasSgemm's op(A)/op(B) arguments
   allow (cuda/math.d:234-235 always passes CUBLAS_OP_N): transA != 0 means A is stored [K][M],
   transB != 0 means B is stored [N][K].  Plans compiled with DOPT_HIP_PLAN_FUSE use it to skip
   the `transpose` kernels that only feed a matmul. */
int dopt_hip_sgemm_t(int transA, int transB, size_t M, size_t N, size_t K, const float *A,
                     const float *B, float *C);
/* `n` independent products in one call, each computed exactly as dopt_hip_sgemm_t computes it (same kernel body, same
   order of summation).  The reference issues one cublasSgemm per matmul (cuda/math.d:234-235); the weight and bias
   gradients of a dense head are products that wait for nothing but the gradient in front of them, and those among
   them that take the small-output kernel or the short column sum share launches here.  No C may overlap an operand
   of another job: the order inside the batch is not kept. */
int dopt_hip_sgemm_batch(int n, const int *transA, const int *transB, const size_t *M, const size_t *N, const size_t *K,
                         const float *const *A, const float *const *B, float *const *C);
/* Names the order in which dopt_hip_sgemm_t adds the K terms of an output element for these flags and dimensions
   (which kernel runs, and where it cuts the reduction): two calls with equal values give equal bits for equal
   operand values, also when one computes the transpose of the other's product, (A B)^T = B^T A^T with M and N
   exchanged; calls with different values may differ in the last bits.  Operands are taken to lie on 16-byte
   boundaries, as every buffer of this library does.  0: the device could not be initialised.  No counterpart in the
   reference, whose plans never rewrite a product; plans compiled with DOPT_HIP_PLAN_FUSE read a transposed
   operand in place only where this says that the values stay what the `transpose` copies would have given. */
uint64_t dopt_hip_sgemm_order(int transA, int transB, size_t M, size_t N, size_t K);
/* C = op(A) * op(B) + u[M,1] * v[1,N], then relu when relu != 0: a dense layer as the reference
   spells it -- matmul(x, W^T) (nnet/layers/dense.d:107) plus the bias broadcast over the rows, which
   is itself a matmul with a ones column (dense.d:143, core/ops/basic.d:370-381), then the relu
   layer -- in one kernel.  u and v may both be null (no rank-one term).  The product, the rank-one
   term, the sum and the relu are each rounded as the four separate kernels round them, so the
   result is identical to running them one after the other.  Used by plans compiled with
   DOPT_HIP_PLAN_FUSE. */
int dopt_hip_sgemm_rank1(int transA, int transB, size_t M, size_t N, size_t K, const float *A,
                         const float *B, const float *u, const float *v, int relu, float *C);
/* C = reluGrad(op(A) * op(B), ., x), i.e. the product where x[M,N] > 0 and zero elsewhere: the input gradient of a
   dense layer (nnet/layers/dense.d:107, differentiated by core/ops/math.d:234-256) passed through the relu in front
   of it (cudnnActivationBackward, cudnn7.d:470).  The mask is applied in the product's epilogue where the
   small-output kernel runs it and by dopt_hip_relu_bwd in place behind it otherwise; either way the values are those
   of dopt_hip_sgemm_t followed by dopt_hip_relu_bwd.  Used by plans compiled with DOPT_HIP_PLAN_FUSE. */
int dopt_hip_sgemm_relu_grad(int transA, int transB, size_t M, size_t N, size_t K, const float *A,
                             const float *B, const float *x, float *C);

typedef struct {
    size_t N, C, H, W;       /* features [N,C,H,W] */
    size_t K, R, S;          /* filters  [K,C,R,S] */
    size_t padH, padW, strideH, strideW;
} dopt_hip_conv_desc;

/* `convolution`: cudnnConvolutionForward at cudnn7.d:154, CUDNN_CONVOLUTION mode (:87): a TRUE
   convolution, y[n,k,p,q] = sum x[n,c,p*sy-ph+r,q*sx-pw+s] * w[k,c,R-1-r,S-1-s]. */
int dopt_hip_conv_fwd(const dopt_hip_conv_desc *d, const float *x, const float *w, float *y);
/* `addBias(convolution(x, w), bias)` in one pass: the two reference kernels (cudnn7.d:154 then
   cudnnAddTensor at cudnn7.d:507) with the bias added where the sums are finished.  Same
   values as the two calls; used by plans compiled with DOPT_HIP_PLAN_FUSE. */
int dopt_hip_conv_fwd_bias(const dopt_hip_conv_desc *d, const float *x, const float *w,
                           const float *bias, float *y);
/* `convolutionFeaturesGrad` (also convolutionTranspose): cudnnConvolutionBackwardData, cudnn7.d:199. */
int dopt_hip_conv_bwd_data(const dopt_hip_conv_desc *d, const float *dy, const float *w, float *dx);
/* Filters packed ahead of the convolutions that read them.  The forward and backward-data kernels
   of 3x3 unit-stride convolutions read the filter in a layout of their own, which the entry points
   above produce on every call; a caller that runs many convolutions per step (a plan) can pack all
   their filters in ONE launch and hand the packed copies over instead.  The reference has no
   counterpart: cuDNN reads [K, C, R, S] directly (cuda/nnet/cudnn7.d:161-175, :229-241).
   dopt_hip_conv_packed_bytes: size of the packed copy for the forward (bwd_data = 0) or the
   backward-data (1) direction, or 0 when that convolution does not take one (the caller then uses
   the unpacked entry points).  A packed copy depends on the descriptor, the direction and the
   device, and is valid until the filter changes.  Layers that run the Winograd F(2x2, 3x3) kernel (pad 1, even
   image sides of 4 and more, whole 16-channel chunks and at least 64 reduction channels, rows in whole 128s or
   in 64s padded by at most a fifth) get the transformed filter G g Gt as their packed copy, 16/9 the size. */
size_t dopt_hip_conv_packed_bytes(const dopt_hip_conv_desc *d, int bwd_data);
/* Which layout that packed copy has, or -1 when there is none: two packed copies of the same filter
   under the same descriptor and with equal layout ids are identical, so a caller needs only one.
   Layout 3 is the filter itself, [K, C, R, S]: the kernel reads it as it lies, dopt_hip_conv_pack_batch
   makes a plain copy, and a caller may skip that and pass the filter as `packed` (it must be 16-byte
   aligned). */
int dopt_hip_conv_packed_layout(const dopt_hip_conv_desc *d, int bwd_data);
int dopt_hip_conv_pack_batch(int n, const dopt_hip_conv_desc *descs, const int *bwd_data,
                             const float *const *w, float *const *packed /* 16-byte aligned */);
/* bias may be null */
int dopt_hip_conv_fwd_bias_packed(const dopt_hip_conv_desc *d, const float *x, const float *packed,
                                  const float *bias, float *y);
int dopt_hip_conv_bwd_data_packed(const dopt_hip_conv_desc *d, const float *dy, const float *packed, float *dx);
/* A convolution result left open: convolutions with few output tiles split their reduction over
   several workgroups and finish with a pass that adds the partial copies (and the bias).  When the
   next reader is a batch norm that reads the whole value anyway, that reader can add the copies
   itself and the finishing pass is dropped.  The *_open entry points below are the packed entry
   points above, except that when the reduction was split they skip the finishing pass and describe
   the partial copies here; the value then MUST be closed by the very next call into this library
   (dopt_hip_split_sum_close, dopt_hip_bn_train_open or dopt_hip_bn_grad_open): the copies live in
   the library's workspace.  splits == 0 means the value is complete and there is nothing to close.
   No counterpart in the reference, where cuDNN owns its workspace (cuda/nnet/cudnn7.d:111). */
typedef struct dopt_hip_split_sum {
    const float *partial; /* [splits][elems], copy s before copy s + 1 */
    int splits;           /* 0: value is complete */
    size_t elems;         /* N * C * inner */
    size_t C, inner;      /* the value is [N, C, inner] */
    const float *bias;    /* per-channel addend of the finished sum, or null */
    float *value;         /* where the finished sum belongs */
    int lanes;            /* 0: the copies are added one after the other (((c0 + c1) + c2) + ...).  L > 0 (an open filter
                             gradient): L interleaved lanes, lane l folding copies l, l + L, l + 2L, ... in four chains
                             (chain j takes every fourth of them, starting from zero), lane value = (ch0 + ch1) + (ch2 + ch3),
                             and the lane values are added in lane order: the order of the filter gradient's own
                             finishing pass.  C, inner and bias are not used then. */
} dopt_hip_split_sum;
int dopt_hip_conv_fwd_bias_packed_open(const dopt_hip_conv_desc *d, const float *x, const float *packed,
                                       const float *bias, float *y, dopt_hip_split_sum *open);
int dopt_hip_conv_bwd_data_packed_open(const dopt_hip_conv_desc *d, const float *dy, const float *packed,
                                       float *dx, dopt_hip_split_sum *open);
/* Backward-data (on a packed filter, as dopt_hip_conv_bwd_data_packed_open; open may be null) and filter gradient
   (as dopt_hip_conv_bwd_filter) of one convolution in one call: cudnnConvolutionBackwardData (cudnn7.d:195) and
   cudnnConvolutionBackwardFilter (cudnn7.d:244) read the same dy and nothing of each other.  For 3x3 unit-stride
   layers of at least 128 input and output channels on rows of 8 .. 64 pixels or 4 x 4 images whose backward-data is
   not a Winograd layer both run as ONE launch, the filter-gradient tiles starting on each compute unit as its
   backward-data tile ends; every other shape runs the two entry points one after the other (a Winograd
   backward-data on 128-row tiles and its filter gradient out of one workspace request, so that both can stay
   open).  dx and dw are bit for bit what the two entry points write.
   open_dw (may be null): where the filter gradient is left as partial copies (the one launch always splits its
   pixels over the compute units), the pass that adds them is skipped and the copies are described there, to be
   closed by the next call like an open dx: dopt_hip_split_sum_close, or dopt_hip_bn_grad_side, whose launch adds
   them on compute units the batch norm leaves idle.  Both open and open_dw may be pending at once. */
int dopt_hip_conv_bwd_pair_packed_open(const dopt_hip_conv_desc *d, const float *dy, const float *packed,
                                       const float *x, float *dx, float *dw, dopt_hip_split_sum *open,
                                       dopt_hip_split_sum *open_dw);
/* Measurement aid (no counterpart in the reference; CUDAPlan.profiler, cuda/package.d:424-431, times whole kernel
   objects): while enabled, every launch of one kernel family is bracketed by two events on the library's queue, so
   its device time is known apart from the split sums and packing the same entry point runs.  probe(1) collects the
   one-launch pairs above, probe(2) the launches of the Winograd kernel (forward and backward-data of 3x3 layers with
   whole 128-row tiles); either starts a fresh collection, probe(0) stops it.  read waits for the launches collected so
   far and returns their number, their summed duration, their FLOPs by the direct algorithm's count (2 N K C 9 P Q per
   product, every tap: what a pair executes; the Winograd kernel executes 16/36 of it) and their algorithmic bytes
   (every operand and result once).  Launches recorded into a HIP graph are not collected. */
int dopt_hip_conv_pair_probe(int enable);
int dopt_hip_conv_pair_probe_read(int *launches, double *total_us, double *flops, double *bytes);
/* value = sum of the copies in order (+ bias): what the closed entry points do themselves. */
int dopt_hip_split_sum_close(const dopt_hip_split_sum *open);
/* `convolutionFiltersGrad`: cudnnConvolutionBackwardFilter, cudnn7.d:244. */
int dopt_hip_conv_bwd_filter(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw);
/* `n` independent filter gradients in one call, each as dopt_hip_conv_bwd_filter computes it (the reference runs one
   cudnnConvolutionBackwardFilter per layer, cudnn7.d:244; none of them reads another's result).  Runs of 2x2-image
   layers share one launch; no dw may overlap another job's operands. */
int dopt_hip_conv_bwd_filter_batch(int n, const dopt_hip_conv_desc *descs, const float *const *dy, const float *const *x,
                                   float *const *dw);

/* ---------------------------------------------------------------------------------------
 * Bandwidth-bound NN ops (fp32, NCHW; `inner` = product of the dims after the channel dim).
 * ------------------------------------------------------------------------------------- */

/* `maxpool`: cudnnPoolingForward, cudnn7.d:303; window = stride = (ph, pw), no padding,
   output dims floor(H/ph) x floor(W/pw) (core/ops/nnet.d:97-107). */
int dopt_hip_maxpool_fwd(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw, const float *x, float *y);
/* `maxpoolGrad`: cudnnPoolingBackward, cudnn7.d:328.  The reference passes (dy, y, x); y is
   recomputed from x here, so it is not an argument.  Ties go to the first maximum of the
   window in row-major order. */
int dopt_hip_maxpool_bwd(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw,
                         const float *dy, const float *x, float *dx);
/* `softmax` over dim 1 of [N, C, inner]: cudnnSoftmaxForward ACCURATE/CHANNEL, cudnn7.d:364;
   arithmetic order of cpu/nnet.d:129-166. */
int dopt_hip_softmax_fwd(size_t N, size_t C, size_t inner, const float *x, float *y);
/* `softmaxGrad`: cudnnSoftmaxBackward, cudnn7.d:397; dx = y * (dy - sum_c dy*y). */
int dopt_hip_softmax_bwd(size_t N, size_t C, size_t inner, const float *dy, const float *y, float *dx);
/* `relu`: cudnnActivationForward RELU / PROPAGATE_NAN, cudnn7.d:433. */
int dopt_hip_relu_fwd(size_t n, const float *x, float *y);
/* `reluGrad`: cudnnActivationBackward, cudnn7.d:471; dx = x > 0 ? dy : 0 (y is not needed). */
int dopt_hip_relu_bwd(size_t n, const float *dy, const float *x, float *dx);
/* `addBias`: cuMemcpy + cudnnAddTensor, cudnn7.d:502-507; y = x + b[c] in one pass. */
int dopt_hip_bias_fwd(size_t N, size_t C, size_t inner, const float *x, const float *b, float *y);
/* `addBiasGrad`: cudnnConvolutionBackwardBias, cudnn7.d:539-540; db[c] = sum_{n,i} dy.  The
   reference passes beta = 1 and so accumulates into its output buffer across executions;
   this computes the plain sum (beta = 0), identical on the first execution. */
int dopt_hip_bias_bwd(size_t N, size_t C, size_t inner, const float *dy, float *db);
/* dopt_hip_bias_bwd for callers that cannot allocate device memory (code recording a HIP graph, tight
   serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels and
   the same result bit for bit, but the per-(channel, image-slice) partial sums of the sliced path
   (rows of at least 256 values) go to a 256 KiB array built into the library for this entry point alone
   (one copy per device, held until the process ends), and the call sets nothing up: no lazy
   initialisation, no allocation, no free, no fill through the runtime.  Needs dopt_hip_init to have run.
   Limit: C * S <= 65536 partial sums, where S = min(64, N, ceil(8 * CUs / C)) -- with 256 compute
   units that is every C <= 65536; beyond it the call fails with DOPT_HIP_ERR_INVALID and launches
   nothing.  All calls on a device share that array (each call overwrites what it reads before reading
   it, so nothing has to be cleared): calls that overlap on one device -- two host threads, two streams
   -- race. */
int dopt_hip_bias_bwd_noalloc(size_t N, size_t C, size_t inner, const float *dy, float *db);

/* `uniform`: curandGenerateUniform at cuda/random.d:74 -- n floats drawn uniformly from (0, 1].
   Counter-based Philox4x32-10: the values depend only on (seed, call, element index); a kernel
   object draws `seed` once (the reference seeds with unpredictableSeed, cuda/random.d:64) and
   passes call = 0, 1, 2, ... on successive executions.  dopt_hip_philox_raw writes the
   generator's 32-bit words themselves (for known-answer tests of the generator). */
int dopt_hip_uniform(uint64_t seed, uint64_t call, size_t n, float *out);
int dopt_hip_philox_raw(uint64_t seed, uint64_t call, size_t n, uint32_t *out);

/* Training-time image augmentation of nnet/data/imagetransformer.d:45-138 (ImageTransformer.getBatch),
   which the reference runs on the host, one image at a time, before the batch is uploaded: pad by
   (jitterY, jitterX) with the image mirrored about its edges, crop an H x W window at (yoff, xoff)
   in the padded image, then reverse rows (flip X) and/or columns (flip Y).  Here the batch is
   already on the device and one kernel writes every output pixel from its source pixel.
   geom: N triples on the device {xoff in [0, 2*jitterX], yoff in [0, 2*jitterY], flags: bit 0 = flip
   X, bit 1 = flip Y}; the caller draws them (the reference uses std.random on the host too). */
int dopt_hip_image_transform(size_t N, size_t C, size_t H, size_t W, size_t jitterX, size_t jitterY,
                             const int32_t *geom, const float *in, float *out);

/* `batchNormTrain`: cudnnBatchNormalizationForwardTraining (spatial), cudnn7.d:608-610.
   packed = [ y (N*C*inner) | newRunMean (C) | newRunVar (C) ] as core/ops/nnet.d:222-225;
   momentum is the op attribute (running = momentum*running + (1-momentum)*batch; the running
   variance takes the unbiased batch estimate); eps = 1e-5f. */
int dopt_hip_bn_train(size_t N, size_t C, size_t inner, double momentum, const float *x,
                      const float *scale, const float *bias, const float *run_mean,
                      const float *run_var, float *packed);
/* `batchNormGrad`: cudnnBatchNormalizationBackward, cudnn7.d:632-634.
   packed = [ dx | dscale (C) | dbias (C) ] as core/ops/nnet.d:232-235; batch statistics are
   recomputed from x as the reference does (it saves none). */
int dopt_hip_bn_grad(size_t N, size_t C, size_t inner, const float *dy, const float *x,
                     const float *scale, float *packed);
/* Fused forms used by plans compiled with DOPT_HIP_PLAN_FUSE; each gives the values of the two
   reference kernels it stands for.
   bn_train_relu: `relu(batchNormTrain(...).y)`: cudnn7.d:608-610 then cudnnActivationForward
   (cudnn7.d:433); the y part of `packed` holds the ReLU output.
   bn_grad_relu: `batchNormGrad(reluGrad(dy, y, .), x, scale)`: cudnnActivationBackward
   (cudnn7.d:471) then cudnn7.d:632-634; dy is dropped where the ReLU output y is not
   positive. */
int dopt_hip_bn_train_relu(size_t N, size_t C, size_t inner, double momentum, const float *x,
                           const float *scale, const float *bias, const float *run_mean,
                           const float *run_var, float *packed);
int dopt_hip_bn_grad_relu(size_t N, size_t C, size_t inner, const float *dy, const float *y,
                          const float *x, const float *scale, float *packed);
/* bn_grad_fused: batchNormGrad with either neighbour folded in.  y (optional) is the ReLU output
   as in bn_grad_relu; dx_sum (optional, C floats) receives the per-channel sum of dx, which is
   `addBiasGrad(dx)` (cudnnConvolutionBackwardBias, cudnn7.d:539) when the batch norm's
   input came from addBias.  dx_sum is summed in a different order than the stand-alone kernel
   sums it (same value up to fp32 rounding). */
int dopt_hip_bn_grad_fused(size_t N, size_t C, size_t inner, const float *dy, const float *y,
                           const float *x, const float *scale, float *packed, float *dx_sum);
/* The same two kernels reading an open convolution result (see dopt_hip_split_sum): x_open->value is
   the batch norm's input x; it is closed on the way (written in full, bit for bit what
   dopt_hip_split_sum_close writes) because the backward pass reads it.  relu != 0: as
   dopt_hip_bn_train_relu.  For the gradient, dy_open->value is dy; keep_dy == 0 says that nothing
   else reads dy, which then need not be written (and is not, where the kernel adds the copies itself). */
int dopt_hip_bn_train_open(size_t N, size_t C, size_t inner, double momentum, const dopt_hip_split_sum *x_open,
                           const float *scale, const float *bias, const float *run_mean, const float *run_var,
                           float *packed, int relu);
int dopt_hip_bn_grad_open(size_t N, size_t C, size_t inner, const dopt_hip_split_sum *dy_open, int keep_dy,
                          const float *y, const float *x, const float *scale, float *packed, float *dx_sum);
/* Batch norm with the 2 x 2 max-pool behind it (`maxpool` with dims [2, 2], cudnn7.d:300-357) in the same
   launch, for [N, C, H, W] with H and W even.  No counterpart in the reference, which runs
   cudnnBatchNormalization* and cudnnPooling* one after the other; results are bit for bit those of the
   separate calls.
   bn_train_pool: packed is what dopt_hip_bn_train (relu == 0) or dopt_hip_bn_train_relu writes, and
   pooled[N, C, H/2, W/2] = maxpool(y).  x_open (optional) is an open convolution result as in
   dopt_hip_bn_train_open; x is ignored then.
   bn_grad_pool: batchNormGrad(reluGrad(maxpoolGrad(dpooled, ., y), y, .), x, scale) where y is the ReLU
   output that was pooled; dx_sum as in dopt_hip_bn_grad_fused.  The [N, C, H, W] gradient of the pool is never
   stored.
   Images of 2 x 2, or of W = 4 .. 128 a power of two, are pooled inside the register-resident kernels;
   other shapes run the pooling kernel as a pass of its own (for the gradient: into `packed`, in place). */
int dopt_hip_bn_train_pool(size_t N, size_t C, size_t H, size_t W, double momentum, const float *x,
                           const dopt_hip_split_sum *x_open, const float *scale, const float *bias,
                           const float *run_mean, const float *run_var, float *packed, int relu, float *pooled);
int dopt_hip_bn_grad_pool(size_t N, size_t C, size_t H, size_t W, const float *dpooled, const float *y,
                          const float *x, const float *scale, float *packed, float *dx_sum);
/* Every form of the batch-norm gradient above in one entry point, plus a sum that rides along.  The tensor is
   [N, C, H, W] (H * W = inner).  Exactly one of dy, dy_open and dpooled says where the incoming gradient is:
   dy as in dopt_hip_bn_grad_fused; dy_open / keep_dy as in dopt_hip_bn_grad_open; dpooled as in
   dopt_hip_bn_grad_pool (y is required then), and when dpooled_open is given as well, dpooled is its value and
   still lies in partial copies, which the kernel adds as it routes them (keep_dy as for dy_open).
   side (may be null, or complete: splits == 0) is a sum that has nothing to do with the batch norm: an open
   filter gradient left by dopt_hip_conv_bwd_pair_packed_open.  Where a register-resident batch-norm kernel runs,
   extra workgroups of the same launch add its copies (bit for bit what dopt_hip_split_sum_close writes); both
   are short bandwidth-bound passes, and one launch costs less than two.  Elsewhere it is closed first by a launch
   of its own.  No counterpart in the reference. */
int dopt_hip_bn_grad_side(size_t N, size_t C, size_t H, size_t W, const float *dy, const dopt_hip_split_sum *dy_open,
                          int keep_dy, const float *dpooled, const dopt_hip_split_sum *dpooled_open, const float *y,
                          const float *x, const float *scale, float *packed, float *dx_sum,
                          const dopt_hip_split_sum *side);
/* Channels of more than 32768 values are normalised by a few workgroups each, which meet once inside the
   kernel; a workgroup polls for its partners at most `polls` times (about a microsecond each; default
   2^21) and then gives up: the kernel still ends, and the next dopt_hip_sync or dopt_hip_copy_d2h
   returns DOPT_HIP_ERR_RUNTIME (the batch-norm results since the previous synchronisation are invalid).
   No counterpart in the reference.  A limit of 0 makes every such call give up unless its partners have
   already arrived (used to test the error path). */
int dopt_hip_bn_wait_limit(unsigned polls);
/* `batchNormInference`: cudnnBatchNormalizationForwardInference, cudnn7.d:650-652; eps = 1e-5. */
int dopt_hip_bn_infer(size_t N, size_t C, size_t inner, const float *x, const float *scale,
                      const float *bias, const float *mean, const float *var, float *y);

/* ---------------------------------------------------------------------------------------
 * Fused multi-tensor optimizer updates.  The reference has no such kernels: dopt.online
 * builds each rule as a graph of pointwise ops with GEMM broadcasts
 * (online/source/dopt/online/{sgd,adam,amsgrad}.d).  These kernels restate those graphs with
 * one fp32 rounding per graph node and no FMA contraction, in place, one launch for all
 * tensors.
 * ------------------------------------------------------------------------------------- */

typedef struct {
    float *w;        /* parameter, updated in place unless skip_w */
    const float *g;  /* gradient */
    float *m;        /* momentum buffer (SGD) / first moment (ADAM, AMSGrad), in place */
    float *v;        /* second moment (ADAM, AMSGrad), in place; NULL for SGD */
    float *vhat;     /* running max (AMSGrad), in place; NULL otherwise */
    size_t n;        /* element count */
    int skip_w;      /* 1: a projection replaces the new value (online/adam.d:66-72), leave w alone */
} dopt_hip_tensor_ref;

/* Builds the device-side chunk table for a fixed set of tensors; reuse it every step. */
int dopt_hip_optim_create(int ntensors, const dopt_hip_tensor_ref *refs, void **handle);
int dopt_hip_optim_destroy(void *handle);
/* online/sgd.d:44-63.  mom' = mom*mu (+|-) lr*g;  w' = w - mom'  (Nesterov: (w + mu*mom') - lr*g). */
int dopt_hip_sgd_step(void *handle, float lr, float mu, int nesterov);
/* online/adam.d:44-63.  *b1, *b2 (host) are the persisted running products beta^t; they are
   advanced here exactly as the graph does (nb = b*beta) and eta is derived from them on the
   host in fp32: eta = (alpha*sqrt(1-nb2))/(1-nb1). */
int dopt_hip_adam_step(void *handle, float alpha, float beta1, float beta2, float eps, float *b1, float *b2);
/* online/amsgrad.d:52-69: ADAM's m', v', w' (w' uses v', as the reference does) plus
   vhat' = max(vhat, OLD v). */
int dopt_hip_amsgrad_step(void *handle, float alpha, float beta1, float beta2, float eps, float *b1, float *b2);

#ifdef __cplusplus
}
#endif
#endif /* DOPT_HIP_H */
