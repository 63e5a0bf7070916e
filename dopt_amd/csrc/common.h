// Internal helpers shared by every translation unit of libdopthip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/dopt_hip.h"

namespace dopt {

// Records the message returned by dopt_hip_last_error() and hands back `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// The library stream (created by dopt_hip_init; lazily initialises device 0 otherwise).
hipStream_t stream();
bool ensure_init();
bool is_initialised();   // dopt_hip_init (or a lazily initialising entry point) has run

// Process-wide scratch memory, grown on demand (the analogue of the single conv workspace at
// cuda/nnet/cudnn7.d:111).  Valid until the next call that asks for more; all users enqueue on
// the one library stream, so consecutive users never overlap.
void *workspace(size_t bytes);
// Changes whenever a workspace is reallocated (its address may have changed): whoever keeps the
// address beyond one call -- a recorded HIP graph -- compares generations before using it again.
unsigned long workspace_generation();
// A convolution that leaves its result open parks partial sums in the workspace until the next call adds
// them up; until open_split_clear, any other request for the workspace fails instead of overwriting them.
void open_split_set(const void *partial);
void open_split_clear(const void *partial);
// The library owns two in-order queues.  Everything enqueues on the main one unless a plan has
// switched to the side queue for a step it overlaps with its main chain (set_lane(1) ... set_lane(0));
// each queue has its own workspace.
void set_lane(int lane);
// While a plan records its kernels into a HIP graph, entry points that would allocate (from the
// driver or from the pool), fill device memory or grow the workspace fail instead (none of these can
// be replayed), and the plan runs its kernels directly.
void set_capturing(bool on);
bool capturing();
int scratch_alloc(void **ptr, size_t bytes);   // pooled block, NOT zero-filled; release with dopt_hip_free
// sgemm.hip: C = op(A) * op(B) (+ colbias[col >> bias_shift] per element when colbias is given and the
// shape takes a kernel with that epilogue; *biased says whether it did).
int sgemm_bias(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B, float *C,
               const float *colbias, int bias_shift, bool *biased);
// sgemm.hip: dw[K][C][3][3] = filter gradient of a 3x3, pad-1 convolution over 2x2 images, from x[N][4C]
// and dy[N][4K] in one launch.  Returns false, with nothing launched, for shapes it does not take.
bool sgemm_fold2x2(size_t C, size_t K, size_t N, const float *x, const float *dy, float *dw, int *rc);
// The same for up to 8 layers in one launch; false, with nothing launched, unless every layer suits that kernel.
bool sgemm_fold2x2_batch(int n, const size_t *C, const size_t *K, const size_t *N, const float *const *x,
                         const float *const *dy, float *const *dw, int *rc);
// conv_smallc.hip: 3x3 pad-1 unit-stride convolutions over at most three input channels.  `done`
// stays false when the shape is not theirs (the caller then uses the general kernels).
bool conv_smallc_takes(const dopt_hip_conv_desc *d);
int conv_smallc_fwd(const dopt_hip_conv_desc *d, const float *x, const float *w, const float *bias, float *y, bool *done);
int conv_smallc_wgrad(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw, bool *done);
// nn.hip: out[c] = sum_{n,i} in[n][c][i] in one launch; false, with nothing launched, for shapes it does not take.
bool channel_sum(size_t N, size_t C, size_t inner, const float *in, float *out, int *rc);
hipStream_t lane_stream(int lane);
// bn.hip: error report of the multi-block batch-norm kernels; call with the queues idle.
int bn_cluster_poll();
// bn.hip: how many such kernels have been enqueued so far (a plan samples it around a recording to learn whether the
// recording holds one), and the note a replay of such a recording leaves for the next synchronisation point.
unsigned long bn_cluster_launches();
void bn_cluster_mark_unchecked();
bool bn_cluster_pending();
// Per-device set-up done inside dopt_hip_init, with the device current: addresses of the file-scope device arrays
// (bn.hip: the records blocks of a channel exchange, filled with "absent"; nn.hip: the scratch of
// dopt_hip_bias_bwd_noalloc), so that no later call has to load a code object, fill memory or wait for the device.
int bn_device_setup();
int nn_device_setup();

// Number of compute units of the active device (256 on MI355X); used to size grids.
int num_cus();

inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// hipRTC: compile `source` (once per distinct `key`) and return the named kernel.
int rtc_get(const std::string &key, const std::string &source, const char *kernel_name, hipFunction_t *fn);
int rtc_compile_only(const std::string &source, const char *arch, std::string *log);
int rtc_launch(hipFunction_t fn, unsigned grid, unsigned block, void **args);

}  // namespace dopt

#define DOPT_HIP_CHECK(expr)                                                                       \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return ::dopt::fail(DOPT_HIP_ERR_RUNTIME, "%s:%d: %s failed: %s", __FILE__, __LINE__,  \
                                #expr, hipGetErrorString(e_));                                     \
    } while (0)

#define DOPT_LAUNCH_CHECK()                                                                        \
    do {                                                                                           \
        hipError_t e_ = hipGetLastError();                                                         \
        if (e_ != hipSuccess)                                                                      \
            return ::dopt::fail(DOPT_HIP_ERR_RUNTIME, "%s:%d: kernel launch failed: %s", __FILE__, \
                                __LINE__, hipGetErrorString(e_));                                  \
    } while (0)

#define DOPT_REQUIRE(cond, ...)                                                                    \
    do {                                                                                           \
        if (!(cond)) return ::dopt::fail(DOPT_HIP_ERR_INVALID, __VA_ARGS__);                       \
    } while (0)

#define DOPT_ENSURE_INIT()                                                                         \
    do {                                                                                           \
        if (!::dopt::ensure_init()) return DOPT_HIP_ERR_RUNTIME;                                   \
    } while (0)
