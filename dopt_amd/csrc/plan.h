// Host-side mirror of the reference's backend plugin interface
// (cuda/source/dopt/cuda/package.d), with HIP in place of CUDA in every name.
#pragma once

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace dopt {

// What a kernel constructor can read off an Operation (core/ops/package.d:52-251).
struct Operation {
    std::string opType;
    std::vector<int> deps;
    std::map<std::string, std::vector<size_t>> sizeAttrs;   // attributes["..."].get!(size_t[]) / size_t
    std::map<std::string, double> doubleAttrs;              // attributes["..."].get!double
    int dtype = DOPT_HIP_F32;
    std::vector<size_t> shape;
    void *value = nullptr;  // variable / constant: its HIPBuffer
    size_t volume() const
    {
        size_t v = 1;
        for (size_t s : shape) v *= s;
        return v;
    }
    size_t bytes() const { return volume() * 4; }
    size_t rank() const { return shape.size(); }
};

struct Graph {
    std::vector<Operation> ops;
    ~Graph();
};

// class CUDABuffer (cuda/package.d:124-251) over the pooled allocator.
class HIPBuffer {
public:
    static std::unique_ptr<HIPBuffer> create(size_t numBytes);  // zero-filled; 0 bytes -> empty buffer
    ~HIPBuffer();
    int set(const void *host, size_t bytes);       // "input buffer is the wrong length."
    int set(const HIPBuffer &other);               // "Mismatch in buffer size"
    int get(void *host, size_t bytes) const;       // "output buffer is the wrong length."
    size_t numBytes() const { return mNumBytes; }
    void *ptr() const { return mPtr; }

private:
    HIPBuffer() = default;
    size_t mNumBytes = 0;
    void *mPtr = nullptr;
};

// interface CUDAKernel (cuda/package.d:68-79)
class HIPKernel {
public:
    virtual ~HIPKernel() = default;
    // inputs[i] is the buffer of op.deps[i]; output is preallocated by the plan.
    virtual int execute(const std::vector<const void *> &inputs, const std::vector<size_t> &inputBytes, void *output,
                        size_t outputBytes) = 0;
    // false: execute() does host work that a replayed HIP graph would skip (a caller-registered kernel
    // may do anything); a plan with such a kernel is never recorded.
    virtual bool replayable() const { return true; }
};

// alias CUDAKernelCtr = CUDAKernel delegate(Operation op) (cuda/package.d:25).  A constructor
// reports failure by returning null after calling dopt::fail().
using HIPKernelCtr = std::function<std::unique_ptr<HIPKernel>(const Graph &graph, int op)>;

int registerHIPKernel(const std::string &opName, HIPKernelCtr ctr);   // throws-equivalent if present
void deregisterHIPKernel(const std::string &opName);
std::vector<std::string> listHIPOperations();
void registerBuiltinKernels();  // idempotent

// class CUDAPlan (cuda/package.d:261-433)
class HIPPlan {
public:
    static int create(Graph *graph, const std::vector<int> &outputs, unsigned flags, std::unique_ptr<HIPPlan> *out);
    ~HIPPlan();
    void cleanup();
    int execute(int nargs, const int *argOps, const void *const *argPtrs, const int *argOnHost, int nrets,
                void *const *rets);
    int result(int op, void **ptr, size_t *bytes) const;
    size_t kernelCount() const { return mSteps.size(); }
    void recordings(size_t *recorded, size_t *replays) const
    {
        size_t n = 0;
        for (const CapturedRun &c : mRuns) n += c.exec != nullptr;
        if (recorded) *recorded = n;
        if (replays) *replays = mReplays;
    }
    size_t bufferBytes() const { return mBufferBytes; }
    std::string profile();
    std::map<std::string, std::pair<double, size_t>> profiler;  // opType -> (microseconds, executions)

private:
    HIPPlan() = default;
    struct Builder;                              // create() in passes (plan.cpp)
    struct Step {
        int op;
        std::string label;                       // profiler key: the opType, or "a+b" for a fused pair
        std::vector<int> inputOps;               // operations whose buffers are the kernel's inputs
        std::vector<int> writes;                 // operations besides `op` whose buffers the kernel fills
        std::unique_ptr<HIPKernel> kernel;
        std::vector<const void *> inputs;
        std::vector<size_t> inputBytes;
        int lane = 0;                            // 1: runs on the side queue, beside the main chain
        bool fenceBefore = false;                // side-queue step: first wait for what the main queue holds so far
        bool joinSide = false;                   // main-queue step that reads a side-queue result
    };
    Graph *mGraph = nullptr;
    unsigned mFlags = 0;
    std::vector<int> mOutputs;
    std::vector<int> mOps;                       // topological order
    std::vector<Step> mSteps;                    // kernels to run, in order
    std::unordered_map<int, void *> mResults;    // op -> buffer
    std::vector<void *> mOwned;                  // buffers to free in cleanup
    // Arguments that arrive as host arrays (cuda/package.d:367-401 uploads them with a blocking copy on every
    // execution): two slots per argument, each a page-locked staging copy and a device copy, used in turn.  The host
    // array is copied into the staging memory before the call returns (the caller may change it at once, as after the
    // reference's blocking copy), the upload runs on the second queue beside the previous execution's kernels, and a
    // slot is reused only after the execution that read it has finished (mArgDone).
    struct HostArg { void *pinned = nullptr; void *dev = nullptr; };
    std::unordered_map<int, HostArg> mHostArgs[2];
    hipEvent_t mArgDone[2] = {nullptr, nullptr};
    bool mArgUsed[2] = {false, false};
    int mArgTurn = 0, mArgPending = -1;
    std::vector<int> mAliasSource;               // per op: the op whose buffer it aliases, or -1
    std::vector<size_t> mAliasOffset;            // per op: byte offset into the aliased buffer
    std::vector<char> mNeeded;                   // per op: its result is consumed
    std::vector<std::pair<hipEvent_t, hipEvent_t>> mEvents;
    std::vector<hipEvent_t> mFences;             // ordering between the two queues, one per crossing
    bool mUsesSide = false;
    struct CapturedRun {
        std::vector<const void *> key;           // argument ops and pointers, return pointers
        hipGraph_t graph;
        hipGraphExec_t exec;                     // null until the second execution with this key
        unsigned long wsGeneration;              // workspace_generation() when it was recorded
        bool clusterKernels = false;             // holds a multi-block batch norm: every launch owes an error check
    };
    std::vector<CapturedRun> mRuns;
    bool mGraphOk = false;
    size_t mReplays = 0;
    int enqueue(int nrets, void *const *rets);
    size_t mBufferBytes = 0;
    bool mClean = false;
    std::vector<void *> mRetDst;                 // scratch of execute(): the return copies
    std::vector<const void *> mRetSrc;
    std::vector<size_t> mRetBytes;
    int resolve(int nargs, const int *argOps, const void *const *argPtrs, const int *argOnHost);
};

}  // namespace dopt
