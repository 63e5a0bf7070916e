/*
 * dopt_hip_plan.h -- C ABI of the host-side mirror of dopt's device-backend plugin interface.
 *
 * In the reference the backend is a D package (cuda/source/dopt/cuda/package.d): a kernel
 * registry keyed by op name, a device buffer class, and a Plan that constructs one kernel object
 * per Operation and executes them in topological order.  No D compiler exists where this library
 * is built, so that host layer is written in C++ (dopt_amd/csrc/plan.{h,cpp}: HIPBuffer,
 * HIPKernel, HIPKernelCtr, registerHIPKernel, deregisterHIPKernel, listHIPOperations, HIPPlan,
 * evaluateHIP -- the reference's names with HIP for CUDA) and exported here so that another
 * language can drive it.  A graph handed over through this header carries exactly what a kernel
 * constructor reads off a dopt `Operation`: the op type, the dependencies, the attribute
 * dictionary and the judged output type.
 *
 * Conventions are those of dopt_hip.h (0 = success, dopt_hip_last_error() for the message).
 */
#ifndef DOPT_HIP_PLAN_H
#define DOPT_HIP_PLAN_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ operation graph */

/* A container of Operation records (core/source/dopt/core/ops/package.d:52-251). */
int dopt_hip_graph_create(void **graph);
int dopt_hip_graph_destroy(void *graph);
/* Adds an operation; `deps` are ids returned by earlier calls; (dtype, shape) is the op's
   outputType as judged by the op definition.  "variable" and "constant" own a zero-filled
   device buffer allocated through the backend's variable allocator (cuda/package.d:56). */
int dopt_hip_graph_add_op(void *graph, const char *op_type, int dtype, int rank, const size_t *shape,
                          int ndeps, const int *deps, int *op_id);
/* attributes["key"] = size_t[] / size_t / double (the Variant payloads the kernels read). */
int dopt_hip_graph_set_attr_sizes(void *graph, int op, const char *key, const size_t *values, int n);
int dopt_hip_graph_set_attr_double(void *graph, int op, const char *key, double value);
/* Device buffer behind a variable/constant (`op.value`), and its size in bytes. */
int dopt_hip_graph_value(void *graph, int op, void **device_ptr, size_t *bytes);
/* Read-back used by custom kernel constructors. */
int dopt_hip_graph_op_type(void *graph, int op, const char **op_type, int *dtype, int *rank,
                           size_t *shape8, int *ndeps);
int dopt_hip_graph_op_dep(void *graph, int op, int index, int *dep);

/* ------------------------------------------------------------------ kernel registry */

/* interface CUDAKernel { void execute(const(CUDABuffer)[] inputs, CUDABuffer output); }
   (cuda/package.d:68-79) as a C record: inputs[i] belongs to op.deps[i]. */
typedef struct {
    void *self;
    int (*execute)(void *self, int ninputs, const void *const *inputs, const size_t *input_bytes,
                   void *output, size_t output_bytes);
    void (*destroy)(void *self); /* may be NULL */
} dopt_hip_kernel;

/* alias CUDAKernelCtr = CUDAKernel delegate(Operation op)  (cuda/package.d:25).  Called once
   per Operation when a plan is constructed; returns non-zero to refuse the operation. */
typedef int (*dopt_hip_kernel_ctor)(void *graph, int op, void *user, dopt_hip_kernel *out);

/* registerCUDAKernel (cuda/package.d:479-485): fails if op_name already has a constructor. */
int dopt_hip_register_kernel(const char *op_name, dopt_hip_kernel_ctor ctor, void *user);
/* deregisterCUDAKernel (cuda/package.d:493-496): removing an unknown name is not an error. */
int dopt_hip_deregister_kernel(const char *op_name);
/* listCUDAOperations (cuda/package.d:504-507): newline-separated names, including "variable"
   and "reshape".  Writes at most buf_bytes (NUL-terminated) and reports the size needed. */
int dopt_hip_list_operations(char *buf, size_t buf_bytes, size_t *needed);

/* ------------------------------------------------------------------ plans */

enum {
    /* Result-preserving rewrites applied when the plan is constructed: */
    DOPT_HIP_PLAN_VIEWS = 1,  /* contiguous slices alias their input; slice(pad(x)) that undoes the
                                 pad aliases x; operations left without a consumer are dropped */
    DOPT_HIP_PLAN_TIMING = 2, /* bracket every kernel with HIP events (CUDAPlan.profiler) */
    DOPT_HIP_PLAN_TIMING_SHAPES = 64, /* with TIMING: profiler keys are "opType@d0xd1x..." (the operation's output
                                 shape), so that layers of one type are told apart */
    DOPT_HIP_PLAN_FUSE = 4,   /* with VIEWS: run adjacent operations as one kernel where the middle value
                                 has no other reader -- addBias(convolution), relu(batchNormTrain.y) and
                                 batchNormGrad(reluGrad) -- with the values of the separate kernels */
    DOPT_HIP_PLAN_GRAPH = 16, /* executions whose arguments and return buffers are all device pointers are
                                 recorded into a HIP graph the second time a given set of pointers is bound
                                 and replayed with one launch from then on (plans with per-kernel timing, the
                                 second queue, a `uniform` operation, or a kernel that allocates stay direct) */
    DOPT_HIP_PLAN_OVERLAP = 8, /* filter gradients, and whatever only they feed, run on a second in-order
                                 queue beside the chain that produces the feature gradients; the queues
                                 are ordered by events where a value crosses, and joined before the
                                 outputs are returned.  Same kernels, same values. */
    DOPT_HIP_PLAN_OVERLAP_LIGHT = 32 /* the same second queue for small work only: a step that moves a few
                                 megabytes and whose value reaches nothing but the plan's outputs (the
                                 weight and bias gradients of dense layers) is enqueued right behind its
                                 producers, on the second queue, instead of where the topological order
                                 put it; it then runs beside the large kernels of the main chain, which
                                 it would otherwise follow one launch latency at a time. */
};

/* With DOPT_HIP_PLAN_DUMP=1 in the environment, dopt_hip_plan_create prints the plan's steps to stderr as they will
   run: position, queue, profiler label, operation id and the operations whose buffers the kernel reads. */

/* new CUDAPlan(outputs) (cuda/package.d:267-312): topological sort, one kernel object per
   operation (constructed through the registry), one zero-filled device buffer per operation
   (`reshape` aliases its dependency, `constant` is uploaded once). */
int dopt_hip_plan_create(void *graph, int noutputs, const int *outputs, unsigned flags, void **plan);
/* CUDAPlan.executeImpl (cuda/package.d:343-423).  args: variable ids with the buffer to use in
   place of the variable's own value for this execution (host pointers are uploaded once per
   execution, device pointers are used directly).  A host array is copied into page-locked memory
   of the plan's own before the call returns - the caller may change it at once, as after the
   reference's blocking cuMemcpyHtoD - and uploaded beside the kernels still queued; the plan keeps
   two such copies (and two device copies) per host argument and uses them in turn.  rets[i]
   (device) receives output i with a device-to-device copy; a NULL entry skips the copy. */
int dopt_hip_plan_execute(void *plan, int nargs, const int *arg_ops, const void *const *arg_ptrs,
                          const int *arg_on_host, int nrets, void *const *rets);
/* The plan-owned result buffer of an operation (valid until the plan is destroyed). */
int dopt_hip_plan_result(void *plan, int op, void **device_ptr, size_t *bytes);
/* Number of kernel executions one plan execution issues, and the plan's device footprint. */
int dopt_hip_plan_stats(void *plan, size_t *kernels, size_t *buffer_bytes);
/* With DOPT_HIP_PLAN_GRAPH: how many argument bindings are currently recorded as HIP graphs, and how
   many executions so far were replays of one. */
int dopt_hip_plan_recordings(void *plan, size_t *recorded, size_t *replays);
/* CUDAPlan.profiler (cuda/package.d:265): accumulated device microseconds per op type as
   "opType usec count\n" lines; needs DOPT_HIP_PLAN_TIMING. */
int dopt_hip_plan_profile(void *plan, char *buf, size_t buf_bytes, size_t *needed);
/* CUDAPlan.cleanup (cuda/package.d:322-338) */
int dopt_hip_plan_destroy(void *plan);

#ifdef __cplusplus
}
#endif
#endif /* DOPT_HIP_PLAN_H */
