// Runtime of libdopthip.so: device/stream ownership, the pooled buffer allocator behind
// HIPBuffer (replaces CUDABuffer's cuMemAlloc + GC.collect() per buffer,
// cuda/source/dopt/cuda/package.d:134-156), copies, events, the process-wide workspace and
// the hipRTC compile-and-cache wrapper (replaces cuda/source/dopt/cuda/nvrtc.d).
#include <hip/hiprtc.h>

#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace dopt {

namespace {

thread_local std::string g_last_error;

struct Runtime {
    std::mutex mu;
    bool ready = false;
    int device = 0;
    int cus = 256;
    std::string arch = "gfx950";
    hipStream_t stream = nullptr;
    hipStream_t side = nullptr;     // second in-order queue for work a plan overlaps with its main chain
    hipEvent_t uploads = nullptr;   // behind the uploads queued beside the main queue (dopt_hip_copy_h2d_beside)
    int lane = 0;                   // which of the two the entry points currently enqueue on
    bool capturing = false;         // a plan is recording its kernels into a HIP graph

    // pool
    std::unordered_map<void *, size_t> live;           // ptr -> class size
    // class size -> free blocks, per queue: a block is reused in the order of the queue whose work
    // last touched it, so only allocations made while that queue is current may take it
    std::map<size_t, std::vector<void *>> cached[2];
    size_t live_bytes = 0, cached_bytes = 0, device_allocs = 0;

    // workspace, one per queue: kernels of the two queues run at the same time
    void *ws[2] = {nullptr, nullptr};
    size_t ws_bytes[2] = {0, 0};
    unsigned long ws_generation = 0;   // bumped whenever a workspace moves: recorded graphs hold its address
    const void *open_split[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};   // per queue: partial copies convolutions left in the workspace for their readers

    // rtc
    std::unordered_map<std::string, hipFunction_t> kernels;
    std::vector<hipModule_t> modules;
};

Runtime &rt()
{
    static Runtime r;
    return r;
}

// Size classes: 8 per power of two (<= 12.5 % internal waste), 256-byte minimum so that every
// block is 256-byte aligned relative to hipMalloc's own alignment.
size_t size_class(size_t bytes)
{
    if (bytes <= 256) return 256;
    int hi = 63 - __builtin_clzll((unsigned long long)(bytes - 1));  // floor(log2(bytes-1))
    size_t step = (size_t)1 << (hi >= 3 ? hi - 3 : 0);
    if (step < 256) step = 256;
    return (bytes + step - 1) / step * step;
}

int init_locked(int device)
{
    Runtime &r = rt();
    if (r.ready) {
        if (device != r.device)
            return fail(DOPT_HIP_ERR_INVALID, "dopt_hip_init: already initialised on device %d", r.device);
        return DOPT_HIP_OK;
    }
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return fail(DOPT_HIP_ERR_RUNTIME, "dopt_hip_init: no HIP device available (%s)",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return fail(DOPT_HIP_ERR_INVALID, "dopt_hip_init: device %d out of range (have %d)", device, count);
    DOPT_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    DOPT_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    r.cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    std::string arch = prop.gcnArchName;  // e.g. "gfx950:sramecc+:xnack-"
    r.arch = arch.substr(0, arch.find(':'));
    if (r.arch != "gfx950")
        return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_init: this library is built for gfx950 only, device is %s",
                    r.arch.c_str());
    DOPT_HIP_CHECK(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking));
    DOPT_HIP_CHECK(hipStreamCreateWithFlags(&r.side, hipStreamNonBlocking));   // same (default) priority
    DOPT_HIP_CHECK(hipEventCreateWithFlags(&r.uploads, hipEventDisableTiming));
    // addresses (and the one-time fill) of the file-scope device arrays: nothing is left for a first call to set up
    if (int rc = bn_device_setup()) return rc;
    if (int rc = nn_device_setup()) return rc;
    r.device = device;
    r.ready = true;
    return DOPT_HIP_OK;
}

}  // namespace

int fail(int code, const char *fmt, ...)
{
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

void clear_error() { g_last_error.clear(); }

bool ensure_init()
{
    Runtime &r = rt();
    if (r.ready) return true;
    std::lock_guard<std::mutex> lk(r.mu);
    return init_locked(0) == DOPT_HIP_OK;
}

bool is_initialised() { return rt().ready; }

hipStream_t stream() { return rt().lane ? rt().side : rt().stream; }
hipStream_t lane_stream(int lane) { return lane ? rt().side : rt().stream; }
void set_lane(int lane) { rt().lane = lane ? 1 : 0; }
void set_capturing(bool on) { rt().capturing = on; }
bool capturing() { return rt().capturing; }
int num_cus() { return rt().cus; }
unsigned long workspace_generation() { return rt().ws_generation; }

void open_split_set(const void *partial)
{
    Runtime &r = rt();
    const void **slot = r.open_split[r.lane];
    if (slot[0] == partial || slot[1] == partial) return;
    slot[slot[0] ? 1 : 0] = partial;   // at most two are pending at once: a backward pair's dx and dw
}
void open_split_clear(const void *partial)
{
    Runtime &r = rt();
    for (const void *&slot : r.open_split[r.lane])
        if (slot == partial) slot = nullptr;
}

void *workspace(size_t bytes)
{
    Runtime &r = rt();
    const int l = r.lane;
    if (r.open_split[l][0] || r.open_split[l][1]) {
        // the previous call left partial sums here for the NEXT call to add up; anything else would overwrite them
        r.open_split[l][0] = r.open_split[l][1] = nullptr;   // report once
        fail(DOPT_HIP_ERR_INVALID, "an open convolution result (dopt_hip_conv_*_packed_open) was not closed by the call "
                                   "that followed it: dopt_hip_split_sum_close, dopt_hip_bn_train_open, dopt_hip_bn_grad_open or dopt_hip_bn_grad_side");
        return nullptr;
    }
    if (bytes <= r.ws_bytes[l]) return r.ws[l];
    if (r.capturing) {   // allocation cannot be recorded; the plan falls back to running its kernels directly
        fail(DOPT_HIP_ERR_UNSUPPORTED, "workspace: cannot grow to %zu bytes while a graph is being captured", bytes);
        return nullptr;
    }
    // Growing: earlier users were enqueued on the same queue, and hipFree waits for the device.
    if (r.ws[l]) (void)hipFree(r.ws[l]);
    r.ws[l] = nullptr;
    r.ws_bytes[l] = 0;
    r.ws_generation++;
    size_t want = size_class(bytes);
    if (hipMalloc(&r.ws[l], want) != hipSuccess) {
        fail(DOPT_HIP_ERR_OOM, "workspace: unable to allocate %zu bytes", want);
        return nullptr;
    }
    r.ws_bytes[l] = want;
    return r.ws[l];
}

// ------------------------------------------------------------------------------- hipRTC

static int rtc_compile(const std::string &source, const char *arch, std::vector<char> *code, std::string *log)
{
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), "dopt_rtc.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        return fail(DOPT_HIP_ERR_RTC, "hiprtcCreateProgram failed");
    std::string archopt = std::string("--offload-arch=") + arch;
    // No FMA contraction: a fused chain must round once per graph node like the op graph it
    // replaces.  Packed fp32 VALU ops are disabled for the whole library.
    const char *opts[] = {archopt.c_str(), "-O3", "-ffp-contract=off", "-Xclang", "-target-feature",
                          "-Xclang", "-packed-fp32-ops"};
    hiprtcResult res = hiprtcCompileProgram(prog, (int)(sizeof(opts) / sizeof(opts[0])), opts);
    size_t log_size = 0;
    hiprtcGetProgramLogSize(prog, &log_size);
    std::string l(log_size, '\0');
    if (log_size) hiprtcGetProgramLog(prog, &l[0]);
    if (log) *log = l;
    if (res != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail(DOPT_HIP_ERR_RTC, "hipRTC compilation failed (%s):\n%s", hiprtcGetErrorString(res), l.c_str());
    }
    if (code) {
        size_t sz = 0;
        hiprtcGetCodeSize(prog, &sz);
        code->resize(sz);
        hiprtcGetCode(prog, code->data());
    }
    hiprtcDestroyProgram(&prog);
    return DOPT_HIP_OK;
}

int rtc_compile_only(const std::string &source, const char *arch, std::string *log)
{
    return rtc_compile(source, arch, nullptr, log);
}

int rtc_get(const std::string &key, const std::string &source, const char *kernel_name, hipFunction_t *fn)
{
    Runtime &r = rt();
    auto it = r.kernels.find(key);
    if (it != r.kernels.end()) {
        *fn = it->second;
        return DOPT_HIP_OK;
    }
    std::vector<char> code;
    int rc = rtc_compile(source, r.arch.c_str(), &code, nullptr);
    if (rc) return rc;
    hipModule_t mod;
    DOPT_HIP_CHECK(hipModuleLoadData(&mod, code.data()));
    r.modules.push_back(mod);
    hipFunction_t f;
    DOPT_HIP_CHECK(hipModuleGetFunction(&f, mod, kernel_name));
    r.kernels[key] = f;
    *fn = f;
    return DOPT_HIP_OK;
}

int rtc_launch(hipFunction_t fn, unsigned grid, unsigned block, void **args)
{
    DOPT_HIP_CHECK(hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, 0, stream(), args, nullptr));
    return DOPT_HIP_OK;
}

}  // namespace dopt

using namespace dopt;

extern "C" {

int dopt_hip_init(int device)
{
    std::lock_guard<std::mutex> lk(rt().mu);
    return init_locked(device);
}

int dopt_hip_shutdown(void)
{
    Runtime &r = rt();
    std::lock_guard<std::mutex> lk(r.mu);
    if (!r.ready) return DOPT_HIP_OK;
    (void)hipStreamSynchronize(r.stream);
    (void)hipStreamSynchronize(r.side);
    for (auto &lane_cache : r.cached) {
        for (auto &kv : lane_cache)
            for (void *p : kv.second) (void)hipFree(p);
        lane_cache.clear();
    }
    r.cached_bytes = 0;
    for (auto &kv : r.live) (void)hipFree(kv.first);
    r.live.clear();
    r.live_bytes = 0;
    for (int l = 0; l < 2; l++) {
        if (r.ws[l]) (void)hipFree(r.ws[l]);
        r.ws[l] = nullptr;
        r.ws_bytes[l] = 0;
    }
    r.ws_generation++;
    r.lane = 0;
    for (hipModule_t m : r.modules) (void)hipModuleUnload(m);
    r.modules.clear();
    r.kernels.clear();
    if (r.uploads) (void)hipEventDestroy(r.uploads);
    r.uploads = nullptr;
    (void)hipStreamDestroy(r.stream);
    (void)hipStreamDestroy(r.side);
    r.stream = r.side = nullptr;
    r.ready = false;
    return DOPT_HIP_OK;
}

const char *dopt_hip_last_error(void) { return g_last_error.c_str(); }

// zero = false: a pooled block without the fill, for scratch that its user overwrites entirely
static int pool_take(void **ptr, size_t bytes, bool zero)
{
    DOPT_REQUIRE(ptr != nullptr, "dopt_hip_malloc: ptr is null");
    *ptr = nullptr;
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_ENSURE_INIT();
    Runtime &r = rt();
    // A block taken while a graph is being recorded would be written by every replay, long after it was
    // handed back and given to someone else: the plan runs its kernels directly instead.
    if (r.capturing)
        return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_malloc: a device allocation cannot be recorded into a graph");
    std::lock_guard<std::mutex> lk(r.mu);
    size_t cls = size_class(bytes);
    void *p = nullptr;
    auto &mine = r.cached[r.lane];
    auto it = mine.find(cls);
    if (it != mine.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        r.cached_bytes -= cls;
    } else {
        hipError_t e = hipMalloc(&p, cls);
        if (e != hipSuccess) {
            // give cached blocks back to the driver and retry once
            (void)hipGetLastError();
            // (blocks of the other queue may still be in use by its kernels: wait for both)
            (void)hipStreamSynchronize(r.stream);
            (void)hipStreamSynchronize(r.side);
            for (auto &lane_cache : r.cached) {
                for (auto &kv : lane_cache)
                    for (void *q : kv.second) (void)hipFree(q);
                lane_cache.clear();
            }
            r.cached_bytes = 0;
            e = hipMalloc(&p, cls);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(DOPT_HIP_ERR_OOM, "HIP memory allocation failed: unable to allocate %zu bytes", bytes);
        }
        r.device_allocs++;
    }
    hipError_t e = zero ? hipMemsetAsync(p, 0, bytes, r.lane ? r.side : r.stream) : hipSuccess;
    if (e != hipSuccess) {
        mine[cls].push_back(p);
        r.cached_bytes += cls;
        return fail(DOPT_HIP_ERR_RUNTIME, "HIP default buffer initialisation failed: %s", hipGetErrorString(e));
    }
    r.live[p] = cls;
    r.live_bytes += cls;
    *ptr = p;
    return DOPT_HIP_OK;
}

int dopt_hip_malloc(void **ptr, size_t bytes) { return pool_take(ptr, bytes, true); }

int dopt_hip_free(void *ptr)
{
    if (!ptr) return DOPT_HIP_OK;
    Runtime &r = rt();
    std::lock_guard<std::mutex> lk(r.mu);
    auto it = r.live.find(ptr);
    DOPT_REQUIRE(it != r.live.end(), "Failed to free HIP device memory: %p was not allocated by dopt_hip_malloc", ptr);
    size_t cls = it->second;
    r.live.erase(it);
    r.live_bytes -= cls;
    r.cached[r.lane][cls].push_back(ptr);
    r.cached_bytes += cls;
    return DOPT_HIP_OK;
}

int dopt_hip_pool_trim(void)
{
    Runtime &r = rt();
    std::lock_guard<std::mutex> lk(r.mu);
    if (!r.ready) return DOPT_HIP_OK;
    DOPT_HIP_CHECK(hipStreamSynchronize(r.stream));
    DOPT_HIP_CHECK(hipStreamSynchronize(r.side));
    for (auto &lane_cache : r.cached) {
        for (auto &kv : lane_cache)
            for (void *p : kv.second) (void)hipFree(p);
        lane_cache.clear();
    }
    r.cached_bytes = 0;
    return DOPT_HIP_OK;
}

int dopt_hip_pool_stats(size_t *live_bytes, size_t *cached_bytes, size_t *device_allocs)
{
    Runtime &r = rt();
    std::lock_guard<std::mutex> lk(r.mu);
    if (live_bytes) *live_bytes = r.live_bytes;
    if (cached_bytes) *cached_bytes = r.cached_bytes;
    if (device_allocs) *device_allocs = r.device_allocs;
    return DOPT_HIP_OK;
}

int dopt_hip_memset(void *dst, int byte_value, size_t bytes)
{
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dst != nullptr, "dopt_hip_memset: dst is null");
    DOPT_ENSURE_INIT();
    if (rt().capturing) return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_memset: a fill cannot be recorded into a graph");
    DOPT_HIP_CHECK(hipMemsetAsync(dst, byte_value, bytes, stream()));
    return DOPT_HIP_OK;
}

int dopt_hip_copy_h2d(void *dst, const void *host_src, size_t bytes)
{
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dst && host_src, "Failed to set contents of HIP buffer: null pointer");
    DOPT_ENSURE_INIT();
    // Pageable host memory: the runtime stages the copy and returns once the source is consumed.
    DOPT_HIP_CHECK(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, stream()));
    DOPT_HIP_CHECK(hipStreamSynchronize(stream()));
    return DOPT_HIP_OK;
}

int dopt_hip_host_alloc(void **host_ptr, size_t bytes)
{
    DOPT_REQUIRE(host_ptr != nullptr, "dopt_hip_host_alloc: null argument");
    DOPT_ENSURE_INIT();
    *host_ptr = nullptr;
    if (bytes == 0) return DOPT_HIP_OK;
    if (hipHostMalloc(host_ptr, bytes, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        *host_ptr = nullptr;
        return fail(DOPT_HIP_ERR_OOM, "page-locked host allocation of %zu bytes failed", bytes);
    }
    return DOPT_HIP_OK;
}

int dopt_hip_host_free(void *host_ptr)
{
    if (!host_ptr) return DOPT_HIP_OK;
    DOPT_ENSURE_INIT();
    DOPT_HIP_CHECK(hipStreamSynchronize(stream()));   // a queued copy may still read it
    DOPT_HIP_CHECK(hipHostFree(host_ptr));
    return DOPT_HIP_OK;
}

int dopt_hip_copy_h2d_async(void *dst, const void *pinned_src, size_t bytes)
{
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dst && pinned_src, "dopt_hip_copy_h2d_async: null pointer");
    DOPT_ENSURE_INIT();
    DOPT_HIP_CHECK(hipMemcpyAsync(dst, pinned_src, bytes, hipMemcpyHostToDevice, stream()));
    return DOPT_HIP_OK;
}

int dopt_hip_copy_h2d_beside(void *dst, const void *pinned_src, size_t bytes)
{
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dst && pinned_src, "dopt_hip_copy_h2d_beside: null pointer");
    DOPT_ENSURE_INIT();
    DOPT_REQUIRE(!rt().capturing, "dopt_hip_copy_h2d_beside: not while a plan records its kernels");
    DOPT_HIP_CHECK(hipMemcpyAsync(dst, pinned_src, bytes, hipMemcpyHostToDevice, lane_stream(1)));
    return DOPT_HIP_OK;
}

int dopt_hip_upload_join(void)
{
    DOPT_ENSURE_INIT();
    DOPT_REQUIRE(!rt().capturing, "dopt_hip_upload_join: not while a plan records its kernels");
    DOPT_HIP_CHECK(hipEventRecord(rt().uploads, lane_stream(1)));
    DOPT_HIP_CHECK(hipStreamWaitEvent(lane_stream(0), rt().uploads, 0));
    return DOPT_HIP_OK;
}

int dopt_hip_copy_d2h(void *host_dst, const void *src, size_t bytes)
{
    if (bytes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(host_dst && src, "Failed to get contents of HIP buffer: null pointer");
    DOPT_ENSURE_INIT();
    DOPT_HIP_CHECK(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, stream()));
    DOPT_HIP_CHECK(hipStreamSynchronize(stream()));
    if (!bn_cluster_pending()) return DOPT_HIP_OK;
    // the report is read with both queues idle (a multi-block batch norm may still run on the other one)
    DOPT_HIP_CHECK(hipStreamSynchronize(lane_stream(0)));
    DOPT_HIP_CHECK(hipStreamSynchronize(lane_stream(1)));
    return bn_cluster_poll();
}

int dopt_hip_copy_d2d(void *dst, const void *src, size_t bytes)
{
    if (bytes == 0 || dst == src) return DOPT_HIP_OK;
    DOPT_REQUIRE(dst && src, "dopt_hip_copy_d2d: null pointer");
    DOPT_ENSURE_INIT();
    DOPT_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream()));
    return DOPT_HIP_OK;
}

int dopt_hip_sync(void)
{
    DOPT_ENSURE_INIT();
    DOPT_HIP_CHECK(hipStreamSynchronize(lane_stream(0)));
    DOPT_HIP_CHECK(hipStreamSynchronize(lane_stream(1)));   // idle unless a plan is overlapping work
    return bn_cluster_poll();
}

void *dopt_hip_stream(void) { return ensure_init() ? (void *)stream() : nullptr; }

int dopt_hip_event_create(void **event)
{
    DOPT_REQUIRE(event != nullptr, "dopt_hip_event_create: event is null");
    DOPT_ENSURE_INIT();
    hipEvent_t ev;
    DOPT_HIP_CHECK(hipEventCreate(&ev));
    *event = (void *)ev;
    return DOPT_HIP_OK;
}

int dopt_hip_event_record(void *event)
{
    DOPT_REQUIRE(event != nullptr, "dopt_hip_event_record: event is null");
    DOPT_HIP_CHECK(hipEventRecord((hipEvent_t)event, stream()));
    return DOPT_HIP_OK;
}

int dopt_hip_event_elapsed_ms(void *start, void *stop, float *ms)
{
    DOPT_REQUIRE(start && stop && ms, "dopt_hip_event_elapsed_ms: null argument");
    DOPT_HIP_CHECK(hipEventSynchronize((hipEvent_t)stop));
    DOPT_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return DOPT_HIP_OK;
}

int dopt_hip_event_sync(void *event)
{
    DOPT_REQUIRE(event != nullptr, "dopt_hip_event_sync: event is null");
    DOPT_HIP_CHECK(hipEventSynchronize((hipEvent_t)event));
    return DOPT_HIP_OK;
}

int dopt_hip_event_destroy(void *event)
{
    if (!event) return DOPT_HIP_OK;
    DOPT_HIP_CHECK(hipEventDestroy((hipEvent_t)event));
    return DOPT_HIP_OK;
}

}  // extern "C"

namespace dopt {

int scratch_alloc(void **ptr, size_t bytes) { return pool_take(ptr, bytes, false); }

}  // namespace dopt
