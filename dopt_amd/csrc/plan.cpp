// HIPBuffer, the kernel registry, the built-in kernel objects and HIPPlan: the host side of the
// backend, mirroring cuda/source/dopt/cuda/package.d (registry :479-507, CUDABuffer :124-251,
// CUDAPlan :261-433) and the kernel classes of cuda/source/dopt/cuda/{math,basic}.d and
// cuda/source/dopt/cuda/nnet/cudnn7.d.  Every kernel object pulls shapes and attributes off its
// Operation in its constructor and makes exactly one call into the kernel library in execute().
//
// Differences from the reference that keep results identical:
//   - no device synchronisation after each kernel (one in-order stream);
//   - a host argument is uploaded once per execution, not once per consumer (package.d:373-381);
//   - buffers come from the pool, with no GC.collect() per allocation (package.d:141);
//   - an operation without a registered kernel is an error instead of a silent host round trip
//     (package.d:81-119): sum, maxElement, argmin and the trigonometric ops have device kernels;
//   - optional rewrites (DOPT_HIP_PLAN_VIEWS) replace copies by aliases.
#include "plan.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <random>

#include <algorithm>
#include <cstring>
#include <functional>
#include <set>

#include "../../include/dopt_hip_plan.h"

namespace dopt {

Graph::~Graph()
{
    for (Operation &o : ops)
        if (o.value) dopt_hip_free(o.value);
}

// ------------------------------------------------------------------------------- HIPBuffer

std::unique_ptr<HIPBuffer> HIPBuffer::create(size_t numBytes)
{
    std::unique_ptr<HIPBuffer> b(new HIPBuffer());
    if (numBytes == 0) return b;  // package.d:144-147
    if (dopt_hip_malloc(&b->mPtr, numBytes) != DOPT_HIP_OK) return nullptr;
    b->mNumBytes = numBytes;
    return b;
}

HIPBuffer::~HIPBuffer()
{
    if (mPtr) dopt_hip_free(mPtr);
}

int HIPBuffer::set(const void *host, size_t bytes)
{
    if (bytes != mNumBytes) return fail(DOPT_HIP_ERR_INVALID, "input buffer is the wrong length.");
    return dopt_hip_copy_h2d(mPtr, host, bytes);
}

int HIPBuffer::set(const HIPBuffer &other)
{
    if (other.mNumBytes != mNumBytes) return fail(DOPT_HIP_ERR_INVALID, "Mismatch in buffer size");
    return dopt_hip_copy_d2d(mPtr, other.mPtr, mNumBytes);
}

int HIPBuffer::get(void *host, size_t bytes) const
{
    if (bytes != mNumBytes) return fail(DOPT_HIP_ERR_INVALID, "output buffer is the wrong length.");
    return dopt_hip_copy_d2h(host, mPtr, bytes);
}

// ------------------------------------------------------------------------------- registry

namespace {

std::unordered_map<std::string, HIPKernelCtr> &kernelCtrs()
{
    static std::unordered_map<std::string, HIPKernelCtr> m;
    return m;
}

using ExecFn = std::function<int(const std::vector<const void *> &, void *)>;

class FnKernel : public HIPKernel {
public:
    explicit FnKernel(ExecFn fn) : mFn(std::move(fn)) {}
    int execute(const std::vector<const void *> &inputs, const std::vector<size_t> &, void *output, size_t) override
    {
        return mFn(inputs, output);
    }

private:
    ExecFn mFn;
};

std::unique_ptr<HIPKernel> make(ExecFn fn) { return std::unique_ptr<HIPKernel>(new FnKernel(std::move(fn))); }

const std::vector<size_t> *sizes_attr(const Operation &op, const char *key)
{
    auto it = op.sizeAttrs.find(key);
    if (it == op.sizeAttrs.end()) {
        fail(DOPT_HIP_ERR_INVALID, "operation '%s' has no attribute '%s'", op.opType.c_str(), key);
        return nullptr;
    }
    return &it->second;
}

bool need_deps(const Operation &op, size_t n)
{
    if (op.deps.size() == n) return true;
    fail(DOPT_HIP_ERR_INVALID, "operation '%s' expects %zu dependencies, has %zu", op.opType.c_str(), n,
         op.deps.size());
    return false;
}

bool need_f32(const Operation &op)
{
    if (op.dtype == DOPT_HIP_F32) return true;
    fail(DOPT_HIP_ERR_UNSUPPORTED, "Element type not supported.");  // cuda/math.d:237-240
    return false;
}

// [N, C, prod(rest)] view used by the cuDNN descriptors (cudnn7.d:339-348, 416-418, 488-492)
void nci(const std::vector<size_t> &shape, size_t *N, size_t *C, size_t *inner)
{
    *N = shape.size() > 0 ? shape[0] : 1;
    *C = shape.size() > 1 ? shape[1] : 1;
    *inner = 1;
    for (size_t i = 2; i < shape.size(); i++) *inner *= shape[i];
}

dopt_hip_conv_desc conv_desc(const std::vector<size_t> &x, const std::vector<size_t> &w, const std::vector<size_t> &pad,
                             const std::vector<size_t> &stride)
{
    dopt_hip_conv_desc d{};
    d.N = x[0]; d.C = x[1]; d.H = x[2]; d.W = x[3];
    d.K = w[0]; d.R = w[2]; d.S = w[3];
    d.padH = pad[0]; d.padW = pad[1]; d.strideH = stride[0]; d.strideW = stride[1];
    return d;
}

bool rank4(const std::vector<size_t> &s, const char *what)
{
    if (s.size() == 4) return true;
    fail(DOPT_HIP_ERR_INVALID, "%s must have rank 4", what);
    return false;
}

std::unique_ptr<HIPKernel> pointwiseCtr(const Graph &g, int id)
{
    const Operation &op = g.ops[id];
    std::string name = op.opType;
    const size_t n = op.volume();
    const int dtype = op.dtype;
    const size_t arity = op.deps.size();
    if (arity != 1 && arity != 2) {
        fail(DOPT_HIP_ERR_INVALID, "pointwise operation '%s' with %zu dependencies", name.c_str(), arity);
        return nullptr;
    }
    return make([=](const std::vector<const void *> &in, void *out) {
        return dopt_hip_pointwise(name.c_str(), dtype, n, in[0], arity == 2 ? in[1] : nullptr, out);
    });
}

void registerBuiltinsOnce()
{
    auto &R = kernelCtrs();
    // cuda/math.d:89-92 plus the ops the reference leaves to its host fallback (core/ops/math.d:75-76)
    for (const char *name : {"add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min", "pow",
                             "atan2", "neg", "abs", "sgn", "exp", "log", "sqrt", "sin", "cos", "tan", "asin", "acos",
                             "atan", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh"})
        R[name] = pointwiseCtr;

    // cuda/math.d:214-247
    R["matmul"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        const auto &a = g.ops[op.deps[0]].shape, &b = g.ops[op.deps[1]].shape;
        if (a.size() != 2 || b.size() != 2 || a[1] != b[0]) {
            fail(DOPT_HIP_ERR_INVALID, "matmul: operands must be rank 2 with matching inner dimension");
            return nullptr;
        }
        const size_t M = a[0], K = a[1], N = b[1];
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_sgemm(M, N, K, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };

    // cpu/math.d:90-247 (host fallback in the reference)
    for (const char *name : {"sum", "maxElement"})
        R[name] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
            const Operation &op = g.ops[id];
            if (!need_deps(op, 1)) return nullptr;
            const auto *axes = sizes_attr(op, "axes");
            if (!axes) return nullptr;
            std::vector<size_t> shape = g.ops[op.deps[0]].shape, ax = *axes;
            std::string name = op.opType;
            const int dtype = op.dtype;
            return make([=](const std::vector<const void *> &in, void *out) {
                return dopt_hip_reduce(name.c_str(), dtype, shape.data(), (int)shape.size(), ax.data(), (int)ax.size(),
                                       in[0], out);
            });
        };
    R["argmin"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1)) return nullptr;
        const auto *axis = sizes_attr(op, "axis");
        if (!axis || axis->size() != 1) return nullptr;
        std::vector<size_t> shape = g.ops[op.deps[0]].shape;
        const size_t ax = (*axis)[0];
        const int dtype = g.ops[op.deps[0]].dtype;
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_argmin(dtype, shape.data(), (int)shape.size(), ax, in[0], (int32_t *)out);
        });
    };

    // cuda/basic.d:31-247
    R["slice"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1)) return nullptr;
        const auto *start = sizes_attr(op, "start");
        if (!start) return nullptr;
        std::vector<size_t> in = g.ops[op.deps[0]].shape, out = op.shape, st = *start;
        return make([=](const std::vector<const void *> &i, void *o) {
            return dopt_hip_slice((int)in.size(), in.data(), out.data(), st.data(), i[0], o);
        });
    };
    R["pad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1)) return nullptr;
        const auto *before = sizes_attr(op, "before");
        if (!before) return nullptr;
        std::vector<size_t> in = g.ops[op.deps[0]].shape, out = op.shape, bf = *before;
        return make([=](const std::vector<const void *> &i, void *o) {
            return dopt_hip_pad((int)in.size(), in.data(), out.data(), bf.data(), i[0], o);
        });
    };
    R["repeat"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1)) return nullptr;
        const auto *reps = sizes_attr(op, "repetitions");
        if (!reps) return nullptr;
        std::vector<size_t> in = g.ops[op.deps[0]].shape, rp = *reps;
        return make([=](const std::vector<const void *> &i, void *o) {
            return dopt_hip_repeat((int)in.size(), in.data(), rp.data(), i[0], o);
        });
    };
    R["transpose"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1)) return nullptr;
        const auto *order = sizes_attr(op, "order");
        if (!order) return nullptr;
        const auto &in = g.ops[op.deps[0]].shape;
        if (in.size() > 2) {
            fail(DOPT_HIP_ERR_UNSUPPORTED, "transpose is only implemented for rank <= 2");  // cpu/basic.d:120
            return nullptr;
        }
        const bool swap = in.size() == 2 && (*order)[0] == 1;
        const size_t rows = in.size() == 2 ? in[0] : 1, cols = in.size() == 2 ? in[1] : op.volume();
        const size_t bytes = op.bytes();
        return make([=](const std::vector<const void *> &i, void *o) {
            if (!swap) return dopt_hip_copy_d2d(o, i[0], bytes);
            return dopt_hip_transpose2d(rows, cols, i[0], o);
        });
    };

    // cuda/nnet/cudnn7.d:113-249
    R["convolution"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        const auto *pad = sizes_attr(op, "padding"), *stride = sizes_attr(op, "stride");
        const auto &x = g.ops[op.deps[0]].shape, &w = g.ops[op.deps[1]].shape;
        if (!pad || !stride || !rank4(x, "convolution features") || !rank4(w, "convolution filters")) return nullptr;
        dopt_hip_conv_desc d = conv_desc(x, w, *pad, *stride);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_conv_fwd(&d, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };
    R["convolutionFeaturesGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, filters]; output = features shape (cudnn7.d:167-169)
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        const auto *pad = sizes_attr(op, "padding"), *stride = sizes_attr(op, "stride");
        const auto &w = g.ops[op.deps[1]].shape;
        if (!pad || !stride || !rank4(op.shape, "convolutionFeaturesGrad output") || !rank4(w, "filters")) return nullptr;
        dopt_hip_conv_desc d = conv_desc(op.shape, w, *pad, *stride);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_conv_bwd_data(&d, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };
    R["convolutionFiltersGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, features]; output = filters shape (cudnn7.d:212-214)
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        const auto *pad = sizes_attr(op, "padding"), *stride = sizes_attr(op, "stride");
        const auto &x = g.ops[op.deps[1]].shape;
        if (!pad || !stride || !rank4(x, "features") || !rank4(op.shape, "convolutionFiltersGrad output")) return nullptr;
        dopt_hip_conv_desc d = conv_desc(x, op.shape, *pad, *stride);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_conv_bwd_filter(&d, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };

    // cudnn7.d:251-333
    R["maxpool"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1) || !need_f32(op)) return nullptr;
        const auto *dims = sizes_attr(op, "dims");
        const auto &x = g.ops[op.deps[0]].shape;
        if (!dims || dims->size() != 2 || !rank4(x, "maxpool features")) return nullptr;
        const size_t N = x[0], C = x[1], H = x[2], W = x[3], ph = (*dims)[0], pw = (*dims)[1];
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_maxpool_fwd(N, C, H, W, ph, pw, (const float *)in[0], (float *)out);
        });
    };
    R["maxpoolGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, y, x] (core/ops/nnet.d:402-407)
        if (!need_deps(op, 3) || !need_f32(op)) return nullptr;
        const auto *dims = sizes_attr(op, "dims");
        const auto &x = g.ops[op.deps[2]].shape;
        if (!dims || dims->size() != 2 || !rank4(x, "maxpoolGrad features")) return nullptr;
        const size_t N = x[0], C = x[1], H = x[2], W = x[3], ph = (*dims)[0], pw = (*dims)[1];
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_maxpool_bwd(N, C, H, W, ph, pw, (const float *)in[0], (const float *)in[2], (float *)out);
        });
    };

    // cudnn7.d:335-404
    R["softmax"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(op.shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_softmax_fwd(N, C, inner, (const float *)in[0], (float *)out);
        });
    };
    R["softmaxGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, y]
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(op.shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_softmax_bwd(N, C, inner, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };

    // cudnn7.d:406-478
    R["relu"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1) || !need_f32(op)) return nullptr;
        const size_t n = op.volume();
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_relu_fwd(n, (const float *)in[0], (float *)out);
        });
    };
    R["reluGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, y, x]
        if (!need_deps(op, 3) || !need_f32(op)) return nullptr;
        const size_t n = op.volume();
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_relu_bwd(n, (const float *)in[0], (const float *)in[2], (float *)out);
        });
    };

    // cudnn7.d:480-545
    R["addBias"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 2) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(op.shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bias_fwd(N, C, inner, (const float *)in[0], (const float *)in[1], (float *)out);
        });
    };
    R["addBiasGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 1) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(g.ops[op.deps[0]].shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bias_bwd(N, C, inner, (const float *)in[0], (float *)out);
        });
    };

    // cudnn7.d:547-654
    R["batchNormTrain"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [x, scale, bias, mean, var]
        if (!need_deps(op, 5) || !need_f32(op)) return nullptr;
        auto it = op.doubleAttrs.find("momentum");
        if (it == op.doubleAttrs.end()) {
            fail(DOPT_HIP_ERR_INVALID, "batchNormTrain has no 'momentum' attribute");
            return nullptr;
        }
        const double momentum = it->second;
        size_t N, C, inner;
        nci(g.ops[op.deps[0]].shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bn_train(N, C, inner, momentum, (const float *)in[0], (const float *)in[1],
                                     (const float *)in[2], (const float *)in[3], (const float *)in[4], (float *)out);
        });
    };
    R["batchNormGrad"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [parentGrad, x, scale]
        if (!need_deps(op, 3) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(g.ops[op.deps[1]].shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bn_grad(N, C, inner, (const float *)in[0], (const float *)in[1], (const float *)in[2],
                                    (float *)out);
        });
    };
    R["batchNormInference"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];  // deps [x, scale, bias, mean, var]
        if (!need_deps(op, 5) || !need_f32(op)) return nullptr;
        size_t N, C, inner;
        nci(op.shape, &N, &C, &inner);
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bn_infer(N, C, inner, (const float *)in[0], (const float *)in[1], (const float *)in[2],
                                     (const float *)in[3], (const float *)in[4], (float *)out);
        });
    };

    // cuda/random.d:47-83: a generator per kernel object, seeded unpredictably at construction
    // (DOPT_HIP_SEED in the environment fixes the seed, for reproducible runs); every execution
    // continues the stream
    R["uniform"] = [](const Graph &g, int id) -> std::unique_ptr<HIPKernel> {
        const Operation &op = g.ops[id];
        if (!need_deps(op, 0) || !need_f32(op)) return nullptr;
        static std::atomic<uint64_t> objects{0};
        uint64_t seed;
        if (const char *fixed = std::getenv("DOPT_HIP_SEED")) {
            seed = std::strtoull(fixed, nullptr, 0);
        } else {
            std::random_device rd;
            seed = ((uint64_t)rd() << 32) ^ (uint64_t)rd();
        }
        seed += 0x9E3779B97F4A7C15ull * objects.fetch_add(1);  // distinct streams for the objects of one process
        const size_t n = op.volume();
        auto call = std::make_shared<uint64_t>(0);
        return make([=](const std::vector<const void *> &, void *out) {
            return dopt_hip_uniform(seed, (*call)++, n, (float *)out);
        });
    };
}

bool is_leaf(const Operation &op) { return op.opType == "variable" || op.opType == "constant"; }

}  // namespace

void registerBuiltinKernels()
{
    static bool done = false;
    if (done) return;
    done = true;
    registerBuiltinsOnce();
}

int registerHIPKernel(const std::string &opName, HIPKernelCtr ctr)
{
    registerBuiltinKernels();
    auto &R = kernelCtrs();
    if (R.find(opName) != R.end())
        return fail(DOPT_HIP_ERR_INVALID, "A HIPKernelCtr is already registered for the operation '%s'", opName.c_str());
    R[opName] = std::move(ctr);
    return DOPT_HIP_OK;
}

void deregisterHIPKernel(const std::string &opName)
{
    registerBuiltinKernels();
    kernelCtrs().erase(opName);
}

std::vector<std::string> listHIPOperations()
{
    registerBuiltinKernels();
    std::vector<std::string> names;
    for (auto &kv : kernelCtrs()) names.push_back(kv.first);
    std::sort(names.begin(), names.end());
    names.push_back("variable");
    names.push_back("reshape");
    return names;
}

// ------------------------------------------------------------------------------- HIPPlan

namespace {

struct Alias {
    int source = -1;     // op whose buffer is aliased
    size_t offset = 0;   // bytes
};

void toposort(const Graph &g, int op, std::vector<char> &seen, std::vector<int> &order)
{
    // iterative depth-first walk, dependencies first (core/ops/package.d:284-311)
    std::vector<std::pair<int, size_t>> stack{{op, 0}};
    if (seen[op]) return;
    seen[op] = 1;
    while (!stack.empty()) {
        auto &top = stack.back();
        const Operation &o = g.ops[top.first];
        if (top.second < o.deps.size()) {
            int d = o.deps[top.second++];
            if (!seen[d]) {
                seen[d] = 1;
                stack.push_back({d, 0});
            }
        } else {
            order.push_back(top.first);
            stack.pop_back();
        }
    }
}


// Kernels of fused pairs (see HIPPlan::create).  `id` is the later operation of the pair, whose
// buffer receives the result.
std::unique_ptr<HIPKernel> make_fused(const Graph &g, int id, int kind, void *extra, std::string *label)
{
    const Operation &op = g.ops[id];
    if (kind == 1) {  // addBias(convolution(x, w), b): inputs [x, w, b]
        const Operation &cv = g.ops[op.deps[0]];
        const auto *pad = sizes_attr(cv, "padding"), *stride = sizes_attr(cv, "stride");
        const auto &x = g.ops[cv.deps[0]].shape, &w = g.ops[cv.deps[1]].shape;
        if (!pad || !stride || !rank4(x, "convolution features") || !rank4(w, "convolution filters")) return nullptr;
        dopt_hip_conv_desc d = conv_desc(x, w, *pad, *stride);
        *label = "convolution+addBias";
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_conv_fwd_bias(&d, (const float *)in[0], (const float *)in[1], (const float *)in[2],
                                          (float *)out);
        });
    }
    if (kind == 2) {  // batchNormTrain whose y part is only read through relu: inputs as batchNormTrain
        auto it = op.doubleAttrs.find("momentum");
        if (it == op.doubleAttrs.end()) {
            fail(DOPT_HIP_ERR_INVALID, "batchNormTrain has no 'momentum' attribute");
            return nullptr;
        }
        const double momentum = it->second;
        size_t N, C, inner;
        nci(g.ops[op.deps[0]].shape, &N, &C, &inner);
        *label = "batchNormTrain+relu";
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bn_train_relu(N, C, inner, momentum, (const float *)in[0], (const float *)in[1],
                                          (const float *)in[2], (const float *)in[3], (const float *)in[4], (float *)out);
        });
    }
    if (kind == 8) {  // batchNormGrad(reluGrad(maxpoolGrad(dp, ., y), y, .), x, scale): inputs [dp, y, x, scale]
        const auto &xs = g.ops[op.deps[1]].shape;
        const size_t N = xs[0], C = xs[1], H = xs[2], W = xs[3];
        *label = std::string("maxpoolGrad+reluGrad+batchNormGrad") + (extra ? "+addBiasGrad" : "");
        return make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_bn_grad_pool(N, C, H, W, (const float *)in[0], (const float *)in[1], (const float *)in[2],
                                         (const float *)in[3], (float *)out, (float *)extra);
        });
    }
    // batchNormGrad, with reluGrad folded in (kind 3: inputs [dy, y, x, scale]; else [dy, x, scale])
    // and/or the bias gradient of the preceding addBias written to `extra`
    size_t N, C, inner;
    nci(g.ops[op.deps[1]].shape, &N, &C, &inner);
    const bool relu = kind == 3;
    *label = std::string(relu ? "reluGrad+" : "") + "batchNormGrad" + (extra ? "+addBiasGrad" : "");
    return make([=](const std::vector<const void *> &in, void *out) {
        const float *dy = (const float *)in[0], *y = relu ? (const float *)in[1] : nullptr;
        const float *x = (const float *)in[relu ? 2 : 1], *scale = (const float *)in[relu ? 3 : 2];
        return dopt_hip_bn_grad_fused(N, C, inner, dy, y, x, scale, (float *)out, (float *)extra);
    });
}

}  // namespace

// HIPPlan::create in passes.  The builder holds what the passes share: per operation, which buffer it
// aliases, which operations' buffers feed its kernel, which fused kernel (if any) computes it, who
// reads it.  `p` is the plan under construction.
struct HIPPlan::Builder {
    const Graph &g;
    HIPPlan *p;
    const std::vector<int> &outputs;
    const unsigned flags;
    const int nops;

    std::vector<Alias> alias;
    // inputsOf[id]: the operations whose buffers feed id's kernel (its deps, unless fused);
    // fusedKind[id]: 1 conv+bias, 2 bn+relu, 3 relugrad+bngrad, 6 matmul with transposes, 7 pointwise chain,
    // 8 maxpoolgrad+relugrad+bngrad, 9 matmul+relugrad, 10 member of a tiny run, 11 sum of squares
    std::vector<std::vector<int>> inputsOf;
    std::vector<int> fusedKind;
    std::vector<std::unique_ptr<HIPKernel>> prebuilt;
    std::vector<std::string> prebuiltLabel;
    // readers, counted among the operations that are live after the alias rewrites
    struct Use { int op; int slot; size_t off; };
    std::vector<char> live;
    std::vector<std::vector<Use>> uses;
    std::vector<std::vector<size_t>> exposed;   // byte offsets at which plan outputs (or aliases of them) expose a buffer
    std::vector<int> biasGradOf;                // batchNormGrad op -> the addBiasGrad op it serves
    std::vector<int> poolOf;                    // batchNormTrain op -> the 2 x 2 maxpool op whose buffer its kernel fills too
    std::vector<int> pairOf;                    // packed convolutionFeaturesGrad op -> the convolutionFiltersGrad op of the same layer
    std::vector<int> pairLead;                  // the operation of such a pair that comes first in the order -> the backward-data op
    std::vector<char> pairLater;                // the operation of such a pair that comes second: no step of its own
    std::vector<char> absorbed;
    std::vector<std::vector<int>> tinyWrites;   // last member of a run of tiny operations -> the other members
    std::vector<char> needed;
    // late: the copy is made right in front of its first reader instead of at the start of the run
    struct Prepack { int op, filter; int bwd; dopt_hip_conv_desc d; void *buf; bool owner, late; };
    void pushPackStep(const std::vector<Prepack> &which);
    std::vector<Prepack> packs;
    std::vector<int> packOf;
    // what foldTransposes made of a matmul (or of the transpose behind one): C[M,N] = op(a) * op(b)
    struct MatmulInfo { bool valid = false; int a = -1, b = -1, tA = 0, tB = 0; size_t M = 0, N = 0, K = 0; };
    std::vector<MatmulInfo> mmInfo;
    // steps that run a convolution on a packed filter (candidates for leaving their result open)
    struct ConvStep { size_t step; int op; int bwd; bool bias; dopt_hip_conv_desc d; const float *packed; int filterIn; };
    std::vector<ConvStep> convSteps;

    Builder(const Graph &graph, HIPPlan *plan, const std::vector<int> &outs, unsigned f)
        : g(graph), p(plan), outputs(outs), flags(f), nops((int)graph.ops.size()), alias((size_t)nops),
          inputsOf((size_t)nops), fusedKind((size_t)nops, 0), prebuilt((size_t)nops), prebuiltLabel((size_t)nops),
          live((size_t)nops, 0), uses((size_t)nops), exposed((size_t)nops), biasGradOf((size_t)nops, -1), poolOf((size_t)nops, -1), pairOf((size_t)nops, -1), pairLead((size_t)nops, -1),
          pairLater((size_t)nops, 0),
          absorbed((size_t)nops, 0), tinyWrites((size_t)nops), needed((size_t)nops, 0), packOf((size_t)nops, -1), mmInfo((size_t)nops)
    {
    }

    int root(int id, size_t *off) const   // the operation whose buffer `id` names, and the byte offset into it
    {
        size_t o = 0;
        while (alias[id].source >= 0) {
            o += alias[id].offset;
            id = alias[id].source;
        }
        *off = o;
        return id;
    }
    bool isOutput(int id) const { return !exposed[id].empty(); }

    int findAliases();
    void countReaders();
    void fusePairs();
    void foldTransposes();
    void fuseDenseLayers();
    void fuseDenseBackward();
    bool plainProduct(int id, MatmulInfo *mi, bool sole_reader) const;
    void formTinyRuns();
    void fuseSquareSums();
    void formChains();
    void absorbBiasGrads();
    void absorbPools();
    void pairBackward();
    std::unique_ptr<HIPKernel> makePooledTrain(int id, std::shared_ptr<dopt_hip_split_sum> open, std::string *label);
    void markNeeded();
    int prepackFilters();
    int allocateBuffers();
    int buildSteps();
    void batchIndependent();
    void openSplitSums();
    void rememberAliases();
    int assignQueues();
    int createEvents();
};

int HIPPlan::Builder::findAliases()
{
    // aliases: reshape always (package.d:295-299); contiguous slices and slice-of-pad under VIEWS
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (op.opType == "reshape") {
            if (op.deps.size() != 1) return fail(DOPT_HIP_ERR_INVALID, "reshape expects one dependency");
            alias[id].source = op.deps[0];
        } else if ((flags & DOPT_HIP_PLAN_VIEWS) && op.opType == "slice" && op.deps.size() == 1) {
            const Operation &src = g.ops[op.deps[0]];
            auto st = op.sizeAttrs.find("start");
            if (st == op.sizeAttrs.end() || st->second.size() != src.rank() || op.rank() != src.rank()) continue;
            const std::vector<size_t> &start = st->second;
            // slice(pad(x)) selecting exactly x
            if (src.opType == "pad" && src.deps.size() == 1) {
                auto bf = src.sizeAttrs.find("before");
                if (bf != src.sizeAttrs.end() && bf->second == start && g.ops[src.deps[0]].shape == op.shape) {
                    alias[id].source = src.deps[0];
                    continue;
                }
            }
            bool contiguous = true;
            for (size_t i = 1; i < src.rank(); i++) contiguous = contiguous && start[i] == 0 && op.shape[i] == src.shape[i];
            if (contiguous && src.rank() > 0) {
                size_t inner = 1;
                for (size_t i = 1; i < src.rank(); i++) inner *= src.shape[i];
                alias[id].source = op.deps[0];
                alias[id].offset = start[0] * inner * 4;
            }
        }
    }
    return DOPT_HIP_OK;
}

void HIPPlan::Builder::countReaders()
{
    // readers are counted among the operations that are live after the alias rewrites
    {
        std::vector<int> work(outputs.begin(), outputs.end());
        while (!work.empty()) {
            int id = work.back();
            work.pop_back();
            if (live[id]) continue;
            live[id] = 1;
            if (alias[id].source >= 0) work.push_back(alias[id].source);
            else for (int d : g.ops[id].deps) work.push_back(d);
        }
    }
    for (int id : p->mOps) {
        if (!live[id] || alias[id].source >= 0) continue;
        const Operation &op = g.ops[id];
        for (size_t j = 0; j < op.deps.size(); j++) {
            size_t off;
            const int r = root(op.deps[j], &off);
            uses[r].push_back({id, (int)j, off});
        }
    }
    // byte offsets at which plan outputs (or aliases of them) expose a buffer
    for (int o : outputs) {
        size_t off;
        const int r = root(o, &off);
        exposed[r].push_back(off);
    }
}

// A pair of operations runs as one kernel when the value between them has no other reader.
void HIPPlan::Builder::fusePairs()
{
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (alias[id].source >= 0) continue;
        if (op.opType == "addBias" && op.deps.size() == 2) {
            const int c = op.deps[0];
            if (g.ops[c].opType == "convolution" && g.ops[c].deps.size() == 2 && alias[c].source < 0 && !isOutput(c) &&
                uses[c].size() == 1 && g.ops[c].dtype == DOPT_HIP_F32) {
                fusedKind[id] = 1;
                inputsOf[id] = {g.ops[c].deps[0], g.ops[c].deps[1], op.deps[1]};
            }
        } else if (op.opType == "relu" && op.deps.size() == 1) {
            size_t off;
            const int b = root(op.deps[0], &off);
            const Operation &bn = g.ops[b];
            if (bn.opType != "batchNormTrain" || bn.deps.size() != 5 || off != 0 || fusedKind[b] ||
                op.volume() != g.ops[bn.deps[0]].volume())
                continue;
            bool ok = true;  // the y part may only feed this relu and the x operand of reluGrad (a sign test)
            for (size_t e : exposed[b]) ok = ok && e >= op.bytes();  // outputs may expose the statistics only
            for (const Use &u : uses[b])
                if (u.off == 0 && !(u.op == id || (g.ops[u.op].opType == "reluGrad" && u.slot == 2))) ok = false;
            if (!ok) continue;
            fusedKind[b] = 2;
            alias[id].source = b;  // the relu output IS the y part now
            alias[id].offset = 0;
        } else if (op.opType == "batchNormGrad" && op.deps.size() == 3) {
            size_t off;
            const int rg = root(op.deps[0], &off);
            const Operation &rgo = g.ops[rg];
            // the fused kernel tests the sign of y where reluGrad tests x: the same thing when y = relu(x)
            const bool pair = rgo.opType == "reluGrad" && rgo.deps.size() == 3 &&
                              g.ops[rgo.deps[1]].opType == "relu" && g.ops[rgo.deps[1]].deps.size() == 1 &&
                              g.ops[rgo.deps[1]].deps[0] == rgo.deps[2];
            if (pair && off == 0 && alias[rg].source < 0 &&
                !isOutput(rg) && uses[rg].size() == 1 && rgo.volume() == g.ops[op.deps[1]].volume()) {
                fusedKind[id] = 3;
                inputsOf[id] = {rgo.deps[0], rgo.deps[1], op.deps[1], op.deps[2]};
                // ... and the gradient of a 2 x 2 max-pool of that relu output in front of the reluGrad: the kernel
                // routes the pooled tensor's gradient itself and the full-size gradient of the pool is never stored
                size_t moff, yoff1, yoff2;
                const int mg = root(rgo.deps[0], &moff);
                const Operation &mgo = g.ops[mg];
                const auto *dims = sizes_attr(mgo, "dims");
                const auto &xs = g.ops[op.deps[1]].shape;
                if (mgo.opType == "maxpoolGrad" && mgo.deps.size() == 3 && moff == 0 && alias[mg].source < 0 && !isOutput(mg) &&
                    uses[mg].size() == 1 && mgo.dtype == DOPT_HIP_F32 && dims && dims->size() == 2 && (*dims)[0] == 2 &&
                    (*dims)[1] == 2 && xs.size() == 4 && xs[2] % 2 == 0 && xs[3] % 2 == 0 && g.ops[mgo.deps[2]].shape == xs &&
                    root(mgo.deps[2], &yoff1) == root(rgo.deps[1], &yoff2) && yoff1 == yoff2) {
                    fusedKind[id] = 8;
                    inputsOf[id] = {mgo.deps[0], rgo.deps[1], op.deps[1], op.deps[2]};
                }
            }
        }
    }
}

void HIPPlan::Builder::foldTransposes()
{
    // matmul reads a transposed operand in place instead of a copy made by `transpose`, and
    // transpose(matmul(A, B)) is computed as matmul(B^T, A^T); the transposes left without a
    // reader drop out.  Only where the product as rewritten adds its terms in the order of the product
    // as written (dopt_hip_sgemm_order): a flag or exchanged dimensions can select another kernel, and
    // a plan with rewrites has to give the bits of the plan without.
    auto is_swap = [&](int t) {
        const Operation &o = g.ops[t];
        if (o.opType != "transpose" || o.deps.size() != 1 || o.rank() != 2 || alias[t].source >= 0) return false;
        auto it = o.sizeAttrs.find("order");
        return it != o.sizeAttrs.end() && it->second.size() == 2 && it->second[0] == 1 && it->second[1] == 0 &&
               o.dtype == DOPT_HIP_F32;
    };
    auto through = [&](int id, bool *flip) {  // the matrix behind a chain of 2-d transposes
        *flip = false;
        while (is_swap(id)) {
            id = g.ops[id].deps[0];
            *flip = !*flip;
        }
        return id;
    };
    auto plain_matmul = [&](int m) {
        const Operation &o = g.ops[m];
        return o.opType == "matmul" && o.deps.size() == 2 && o.rank() == 2 && o.dtype == DOPT_HIP_F32 &&
               alias[m].source < 0;
    };
    struct Fold { int a, b; bool tA, tB; size_t M, N, K; bool same_order; };
    auto fold_of = [&](int mm, bool outT) {   // the product `mm` (or its transpose) on the matrices behind the transposes
        Fold f{};
        f.a = through(g.ops[mm].deps[0], &f.tA);
        f.b = through(g.ops[mm].deps[1], &f.tB);
        f.M = g.ops[mm].shape[0];
        f.N = g.ops[mm].shape[1];
        f.K = g.ops[g.ops[mm].deps[0]].shape[1];
        const uint64_t as_written = dopt_hip_sgemm_order(0, 0, f.M, f.N, f.K);
        if (outT) {  // (A B)^T = B^T A^T
            std::swap(f.a, f.b);
            const bool na = !f.tB, nb = !f.tA;
            f.tA = na;
            f.tB = nb;
            std::swap(f.M, f.N);
        }
        f.same_order = as_written != 0 && dopt_hip_sgemm_order(f.tA, f.tB, f.M, f.N, f.K) == as_written;
        return f;
    };
    auto feeds_a_transpose_only = [&](int mm) {
        return uses[mm].size() == 1 && is_swap(uses[mm][0].op) && !isOutput(mm);
    };
    for (int id : p->mOps) {
        if (!live[id]) continue;
        int mm = id;
        bool outT = false;  // compute the transpose of the product
        if (is_swap(id) && plain_matmul(g.ops[id].deps[0]) && feeds_a_transpose_only(g.ops[id].deps[0])) {
            mm = g.ops[id].deps[0];
            outT = true;
        } else if (!plain_matmul(id)) {
            continue;
        }
        if (!outT && fusedKind[id]) continue;
        if (!outT && feeds_a_transpose_only(mm) && fold_of(mm, true).same_order) continue;  // folded into its transpose
        const Fold f = fold_of(mm, outT);
        if (!f.same_order) continue;
        if (!outT && f.a == g.ops[mm].deps[0] && f.b == g.ops[mm].deps[1]) continue;  // nothing to fold
        int a = f.a, b = f.b;
        bool tA = f.tA, tB = f.tB;
        size_t M = f.M, N = f.N, K = f.K;
        fusedKind[id] = 6;
        inputsOf[id] = {a, b};
        const int ta = tA, tb = tB;
        mmInfo[id].valid = true;
        mmInfo[id].a = a; mmInfo[id].b = b; mmInfo[id].tA = ta; mmInfo[id].tB = tb;
        mmInfo[id].M = M; mmInfo[id].N = N; mmInfo[id].K = K;
        prebuilt[id] = make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_sgemm_t(ta, tb, M, N, K, (const float *)in[0], (const float *)in[1], (float *)out);
        });
        prebuiltLabel[id] = outT ? "matmul+transpose" : "matmul";
    }
}

// A dense layer as the reference builds it: add(matmul(x, W^T), matmul(ones[m,1], bias[1,n])), usually
// followed by relu.  When the product and the broadcast have no other reader they run as one kernel
// (dopt_hip_sgemm_rank1); when, besides that, the sum is only read by a relu and by the x operand of
// reluGrad (a sign test, and sign(relu(x)) = sign(x) where it matters), the kernel clamps as well
// and the relu becomes an alias of its output - the same arrangement as batch norm + relu above.
void HIPPlan::Builder::fuseDenseLayers()
{
    auto plain_product = [&](int id, MatmulInfo *mi) { return plainProduct(id, mi, true); };   // a matmul this pass may absorb
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (!live[id] || alias[id].source >= 0 || fusedKind[id] || op.opType != "add" || op.deps.size() != 2 ||
            op.rank() != 2 || op.dtype != DOPT_HIP_F32 || op.volume() == 0)
            continue;
        for (int order = 0; order < 2; order++) {
            // either operand may arrive through a reshape (repeat(bias, m) ends in one): look at the buffer's owner
            size_t poff, qoff;
            const int pid = root(op.deps[(size_t)order], &poff), qid = root(op.deps[(size_t)(1 - order)], &qoff);
            MatmulInfo prod, outer;
            if (pid == qid || poff != 0 || qoff != 0 || !plain_product(pid, &prod) || !plain_product(qid, &outer)) continue;
            if (outer.K != 1 || outer.tA || outer.tB || prod.K == 0 || fusedKind[qid]) continue;   // u[M,1] * v[1,N] as written
            if (prod.M != op.shape[0] || prod.N != op.shape[1] || outer.M != prod.M || outer.N != prod.N) continue;
            // relu behind it?
            int relu_op = -1;
            bool clamp = !isOutput(id);
            for (const Use &u : uses[id]) {
                const Operation &r = g.ops[u.op];
                if (u.off != 0) clamp = false;
                else if (r.opType == "relu" && r.deps.size() == 1 && r.volume() == op.volume() && alias[u.op].source < 0 &&
                         !fusedKind[u.op] && relu_op < 0)
                    relu_op = u.op;
                else if (!(r.opType == "reluGrad" && u.slot == 2)) clamp = false;
            }
            clamp = clamp && relu_op >= 0;
            fusedKind[id] = 8;
            inputsOf[id] = {prod.a, prod.b, outer.a, outer.b};
            const MatmulInfo mi = prod;
            const int relu = clamp ? 1 : 0;
            prebuilt[id] = make([=](const std::vector<const void *> &in, void *out) {
                return dopt_hip_sgemm_rank1(mi.tA, mi.tB, mi.M, mi.N, mi.K, (const float *)in[0], (const float *)in[1],
                                            (const float *)in[2], (const float *)in[3], relu, (float *)out);
            });
            prebuiltLabel[id] = clamp ? "matmul+broadcast+relu" : "matmul+broadcast";
            prebuilt[pid].reset();   // the product no longer runs on its own
            prebuiltLabel[pid].clear();
            fusedKind[pid] = 0;
            if (clamp) {
                alias[relu_op].source = id;   // the relu output IS this buffer now
                alias[relu_op].offset = 0;
            }
            break;
        }
    }
}

// A rank-2 fp32 product as this pass may read it: what foldTransposes made of it, or the matmul as written.
// sole_reader: only a product whose value has exactly one reader and is no plan output (it can be absorbed).
bool HIPPlan::Builder::plainProduct(int id, MatmulInfo *mi, bool sole_reader) const
{
    if (alias[id].source >= 0 || g.ops[id].dtype != DOPT_HIP_F32 || g.ops[id].rank() != 2) return false;
    if (sole_reader && (isOutput(id) || uses[id].size() != 1)) return false;
    if (fusedKind[id] == 6 && mmInfo[id].valid) {
        *mi = mmInfo[id];
        return true;
    }
    const Operation &o = g.ops[id];
    if (fusedKind[id] || o.opType != "matmul" || o.deps.size() != 2) return false;
    const Operation &l = g.ops[o.deps[0]], &r = g.ops[o.deps[1]];
    if (l.rank() != 2 || r.rank() != 2 || l.dtype != DOPT_HIP_F32 || r.dtype != DOPT_HIP_F32) return false;
    mi->valid = true;
    mi->a = o.deps[0]; mi->b = o.deps[1]; mi->tA = mi->tB = 0;
    mi->M = o.shape[0]; mi->N = o.shape[1]; mi->K = l.shape[1];
    return true;
}

// reluGrad(matmul(dz, W), y, x): the input gradient of a dense layer (nnet/layers/dense.d, differentiated by
// core/ops/math.d:234-256) through the relu in front of it - a launch of its own for a few microseconds of work.
// When the product has no other reader it runs with the mask in its epilogue (dopt_hip_sgemm_relu_grad); the values
// do not change.  (The bias gradient next to it, matmul(ones, dz), could be summed by the weight-gradient product on
// the way, but not in the order the ones-vector product adds it: that would make plans with and without the rewrites
// differ in the last bit of every bias, so it stays a kernel of its own.)
void HIPPlan::Builder::fuseDenseBackward()
{
    // Which values the kernels as rewritten so far still read: a reluGrad that a batch-norm gradient reads around
    // (fusePairs) is dead, and the product in front of it now feeds that kernel - it must stay what it is.
    std::vector<char> read((size_t)nops, 0);
    for (int x : p->mOps) {
        if (!live[x] || alias[x].source >= 0) continue;
        for (int d : inputsOf[x]) {
            size_t off;
            read[root(d, &off)] = 1;
        }
    }
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (!live[id] || alias[id].source >= 0 || op.dtype != DOPT_HIP_F32 || op.volume() == 0) continue;
        if (!read[id] && !isOutput(id)) continue;
        if (!fusedKind[id] && op.opType == "reluGrad" && op.deps.size() == 3 && op.rank() == 2) {
            size_t off;
            const int pid = root(op.deps[0], &off);
            MatmulInfo mi;
            if (off != 0 || !plainProduct(pid, &mi, true) || mi.K == 0 || mi.M != op.shape[0] || mi.N != op.shape[1] ||
                g.ops[op.deps[2]].volume() != op.volume() || g.ops[op.deps[2]].dtype != DOPT_HIP_F32)
                continue;
            fusedKind[id] = 9;
            inputsOf[id] = {mi.a, mi.b, op.deps[2]};
            prebuilt[id] = make([=](const std::vector<const void *> &in, void *out) {
                return dopt_hip_sgemm_relu_grad(mi.tA, mi.tB, mi.M, mi.N, mi.K, (const float *)in[0], (const float *)in[1],
                                                (const float *)in[2], (float *)out);
            });
            prebuiltLabel[id] = "matmul+reluGrad";
            prebuilt[pid].reset();   // the product no longer runs on its own
            prebuiltLabel[pid].clear();
            fusedKind[pid] = 0;
        }
    }
}

// Runs of operations on tiny tensors (a softmax over ten classes, the loss behind it, the scalars of an update rule):
// each would be a kernel that lasts as long as the gap between two kernels.  Walking the order, operations that
// dopt_hip_tiny_graph can compute (every tensor involved of at most DOPT_HIP_TINY_ELEMS fp32 values) collect into a
// run; an operation outside that reads a member ends it, so the run can stand where its last member stood: all it
// reads is older, all that reads it comes later.  The run is one step; every member keeps its buffer and gets its
// value there, computed as its own kernel computes it.
void HIPPlan::Builder::formTinyRuns()
{
    const size_t cap = DOPT_HIP_TINY_ELEMS;
    // operations whose values the plan as rewritten so far still computes (a product that a dense-layer kernel absorbed
    // is read by nobody): reachable from the outputs through what each kernel reads.  A run's step stands where its last
    // member does, so a member nobody needs must not be the one to carry it.
    std::vector<char> read((size_t)nops, 0);
    {
        std::vector<int> work(outputs.begin(), outputs.end());
        while (!work.empty()) {
            const int id = work.back();
            work.pop_back();
            if (read[id]) continue;
            read[id] = 1;
            if (alias[id].source >= 0) work.push_back(alias[id].source);
            else for (int d : inputsOf[id]) work.push_back(d);
        }
    }
    auto small_f32 = [&](int id) { return g.ops[id].dtype == DOPT_HIP_F32 && g.ops[id].volume() >= 1 && g.ops[id].volume() <= cap; };
    // what a member is to the kernel; false when it cannot be one
    auto describe = [&](int id, dopt_hip_tiny_node *nd, int (&operands)[2]) -> bool {
        const Operation &o = g.ops[id];
        if (!live[id] || alias[id].source >= 0 || fusedKind[id] || prebuilt[id] || !small_f32(id)) return false;
        if (!read[id]) return false;
        for (int d : o.deps)
            if (!small_f32(d)) return false;
        *nd = dopt_hip_tiny_node{};
        nd->n = (int)o.volume();
        nd->b = -1;
        operands[0] = operands[1] = -1;
        if (o.opType == "reluGrad" && o.deps.size() == 3) {
            for (const Use &u : uses[id])
                if (fusedKind[u.op] == 3 || fusedKind[u.op] == 8) return false;   // that batchNormGrad reads dy and y itself
            if (g.ops[o.deps[0]].volume() != o.volume() || g.ops[o.deps[2]].volume() != o.volume()) return false;
            nd->kind = DOPT_HIP_TINY_POINTWISE;
            nd->op = dopt_hip_pointwise_index("reluGrad");
            operands[0] = o.deps[0];
            operands[1] = o.deps[2];
            return true;
        }
        if (o.opType == "matmul" && o.deps.size() == 2 && o.rank() == 2) {   // [m,1] x [1,n]: a column times a row
            const Operation &l = g.ops[o.deps[0]], &r = g.ops[o.deps[1]];
            if (l.rank() != 2 || r.rank() != 2 || l.shape[1] != 1 || r.shape[0] != 1) return false;
            nd->kind = DOPT_HIP_TINY_POINTWISE;
            nd->op = dopt_hip_pointwise_index("mul");
            nd->a_kind = 2;
            nd->b_kind = 3;
            nd->dims[0] = (int)o.shape[1];
            operands[0] = o.deps[0];
            operands[1] = o.deps[1];
            return true;
        }
        const int arity = o.opType == "relu" ? 1 : dopt_hip_pointwise_arity(o.opType.c_str());
        if (arity > 0 && o.opType != "reluGrad") {
            if (arity != (int)o.deps.size()) return false;
            for (int d : o.deps)
                if (g.ops[d].volume() != o.volume()) return false;
            nd->kind = DOPT_HIP_TINY_POINTWISE;
            nd->op = dopt_hip_pointwise_index(o.opType.c_str());
            operands[0] = o.deps[0];
            if (arity == 2) operands[1] = o.deps[1];
            return nd->op >= 0;
        }
        if ((o.opType == "sum" || o.opType == "maxElement") && o.deps.size() == 1) {
            const auto *axes = sizes_attr(o, "axes");
            const auto &sh = g.ops[o.deps[0]].shape;
            if (!axes || axes->empty() || sh.empty() || sh.size() > 16) return false;
            std::vector<char> red(sh.size(), 0);
            for (size_t a : *axes) {
                if (a >= sh.size() || red[a]) return false;
                red[a] = 1;
            }
            size_t first = sh.size(), last = 0;
            for (size_t i = 0; i < sh.size(); i++)
                if (red[i]) { first = std::min(first, i); last = i; }
            for (size_t i = first; i <= last; i++)
                if (!red[i]) return false;   // more than one run of reduced axes: passes with a temporary in between
            size_t outer = 1, R = 1, inner = 1;
            for (size_t i = 0; i < first; i++) outer *= sh[i];
            for (size_t i = first; i <= last; i++) R *= sh[i];
            for (size_t i = last + 1; i < sh.size(); i++) inner *= sh[i];
            nd->kind = DOPT_HIP_TINY_REDUCE;
            nd->op = o.opType == "sum" ? 0 : 1;
            nd->dims[0] = (int)outer; nd->dims[1] = (int)R; nd->dims[2] = (int)inner;
            operands[0] = o.deps[0];
            return outer * inner == o.volume();
        }
        if ((o.opType == "softmax" && o.deps.size() == 1) || (o.opType == "softmaxGrad" && o.deps.size() == 2)) {
            if (o.rank() < 2) return false;
            size_t N, C, inner;
            nci(o.shape, &N, &C, &inner);
            if (inner == 1 && C >= 64) return false;   // such rows take the wavefront-per-row kernels
            for (int d : o.deps)
                if (g.ops[d].volume() != o.volume()) return false;
            nd->kind = o.opType == "softmax" ? DOPT_HIP_TINY_SOFTMAX : DOPT_HIP_TINY_SOFTMAX_GRAD;
            nd->dims[0] = (int)N; nd->dims[1] = (int)C; nd->dims[2] = (int)inner;
            operands[0] = o.deps[0];
            if (o.deps.size() == 2) operands[1] = o.deps[1];
            return true;
        }
        if (o.opType == "repeat" && o.deps.size() == 1) {
            const auto *reps = sizes_attr(o, "repetitions");
            const auto &sh = g.ops[o.deps[0]].shape;
            if (!reps || reps->size() != sh.size() || sh.size() > 4) return false;
            nd->kind = DOPT_HIP_TINY_REPEAT;
            for (int d = 0; d < 4; d++) nd->dims[d] = nd->reps[d] = 1;
            const size_t lead = 4 - sh.size();
            for (size_t i = 0; i < sh.size(); i++) {
                nd->dims[lead + i] = (int)sh[i];
                nd->reps[lead + i] = (int)(*reps)[i];
            }
            operands[0] = o.deps[0];
            return true;
        }
        return false;
    };
    struct Member { int op; dopt_hip_tiny_node nd; int operands[2]; };
    std::vector<Member> run;
    std::vector<char> inRun((size_t)nops, 0);
    auto close = [&]() {
        if (run.size() >= 2) {
            // buffers: the members' own, and whatever else they read (by owner of the buffer, with the byte offset in the node)
            std::vector<int> slots;
            auto slot_of = [&](int owner) {
                for (size_t k = 0; k < slots.size(); k++)
                    if (slots[k] == owner) return (int)k;
                slots.push_back(owner);
                return (int)slots.size() - 1;
            };
            std::vector<dopt_hip_tiny_node> nodes;
            bool fits = true;
            for (Member &m : run) {
                dopt_hip_tiny_node nd = m.nd;
                nd.dst = slot_of(m.op);
                for (int k = 0; k < 2; k++) {
                    if (m.operands[k] < 0) continue;
                    size_t off;
                    const int r = root(m.operands[k], &off);
                    if (off > 0x7fffffffu) fits = false;
                    (k == 0 ? nd.a : nd.b) = slot_of(r);
                    (k == 0 ? nd.a_offset : nd.b_offset) = (int)off;
                }
                nodes.push_back(nd);
            }
            if (fits && slots.size() <= (size_t)DOPT_HIP_TINY_SLOTS && nodes.size() <= (size_t)DOPT_HIP_TINY_NODES) {
                const int last = run.back().op;
                for (const Member &m : run) {
                    fusedKind[m.op] = 10;
                    if (m.op != last) absorbed[m.op] = 1;   // keeps its buffer, filled by the run's kernel
                }
                // every buffer is an input of the step (the members' too: that is what keeps them allocated), except the
                // last member's, which is the step's output
                std::vector<int> ins;
                std::vector<int> slotIn(slots.size(), -1);
                for (size_t k = 0; k < slots.size(); k++)
                    if (slots[k] != last) {
                        slotIn[k] = (int)ins.size();
                        ins.push_back(slots[k]);
                    }
                inputsOf[last] = ins;
                tinyWrites[last].clear();
                for (const Member &m : run)
                    if (m.op != last) tinyWrites[last].push_back(m.op);
                const int nslots = (int)slots.size();
                prebuilt[last] = make([=](const std::vector<const void *> &in, void *out) {
                    void *ptrs[DOPT_HIP_TINY_SLOTS];
                    for (int k = 0; k < nslots; k++) ptrs[k] = slotIn[(size_t)k] >= 0 ? const_cast<void *>(in[(size_t)slotIn[(size_t)k]]) : out;
                    return dopt_hip_tiny_graph(nslots, ptrs, (int)nodes.size(), nodes.data());
                });
                prebuiltLabel[last] = "tiny*" + std::to_string(nodes.size());
            }
        }
        for (const Member &m : run) inRun[m.op] = 0;
        run.clear();
    };
    for (int id : p->mOps) {
        if (!live[id]) continue;
        Member m{};
        m.op = id;
        if (describe(id, &m.nd, m.operands)) {
            if (run.size() >= (size_t)DOPT_HIP_TINY_NODES || run.size() * 3 + 3 > (size_t)DOPT_HIP_TINY_SLOTS) close();
            run.push_back(m);
            inRun[id] = 1;
            continue;
        }
        if (alias[id].source >= 0) continue;   // a view: its readers are looked at themselves
        bool reads = false;
        for (int d : inputsOf[id]) {
            size_t off;
            reads = reads || inRun[root(d, &off)];
        }
        if (reads) close();
    }
    close();
}

// sum(mul(x, x)) - the L2 penalty of a parameter (`weightDecay * sum(filters * filters)`, nnet/layers/conv.d:117) and the
// squared norms of nnet/lipschitz.d - where nothing else reads the product: one pass over x that squares on load
// (dopt_hip_reduce_squares), the product rounded to fp32 before it is added and the sums in the reduction's own order,
// so the value is the one the two kernels give; the product is never stored.  Tensors small enough for a tiny run have
// been taken by one already (DOPT_HIP_PLAN_FUSE).
void HIPPlan::Builder::fuseSquareSums()
{
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (!live[id] || alias[id].source >= 0 || fusedKind[id] || prebuilt[id] || op.opType != "sum" || op.deps.size() != 1 ||
            op.dtype != DOPT_HIP_F32 || op.volume() == 0)
            continue;
        const auto *axes = sizes_attr(op, "axes");
        size_t off;
        const int m = root(op.deps[0], &off);
        const Operation &mo = g.ops[m];
        if (!axes || off != 0 || mo.opType != "mul" || mo.deps.size() != 2 || mo.deps[0] != mo.deps[1] || mo.dtype != DOPT_HIP_F32 ||
            !live[m] || fusedKind[m] || prebuilt[m] || isOutput(m) || uses[m].size() != 1 || uses[m][0].op != id ||
            g.ops[mo.deps[0]].dtype != DOPT_HIP_F32 || g.ops[mo.deps[0]].volume() != mo.volume() ||
            g.ops[op.deps[0]].volume() != mo.volume())
            continue;
        const std::vector<size_t> shape = g.ops[op.deps[0]].shape, ax = *axes;
        // one run of adjacent reduced axes: the reduction is one pass (several runs go through temporaries or a kernel
        // of their own, and gain nothing from squaring on load)
        std::vector<char> red(shape.size(), 0);
        bool valid = !ax.empty() && shape.size() <= 16;
        for (size_t a : ax) {
            if (a >= shape.size() || red[a]) { valid = false; break; }
            red[a] = 1;
        }
        int runs = 0;
        for (size_t i = 0; valid && i < shape.size(); i++)
            if (red[i] && (i == 0 || !red[i - 1])) runs++;
        if (!valid || runs != 1) continue;
        fusedKind[id] = 11;
        inputsOf[id] = {mo.deps[0]};
        prebuilt[id] = make([=](const std::vector<const void *> &in, void *out) {
            return dopt_hip_reduce_squares(shape.data(), (int)shape.size(), ax.data(), (int)ax.size(), (const float *)in[0],
                                           (float *)out);
        });
        prebuiltLabel[id] = "mul+sum";
    }
}

void HIPPlan::Builder::formChains()
{
    // Pointwise chains: a pointwise operation whose value is read only by pointwise operations
    // of one chain (and by no plan output) is computed inside that chain's kernel and never
    // stored; an operand of the form repeat(one-element tensor) is read from the element itself.
    // Walking consumers before producers, an operation joins the chain all its readers belong to
    // or starts a chain of its own.
    // What may be a node: the pointwise operations; relu and reluGrad(dy, y, x) (a node of dy and x),
    // unless a batch-norm fusion above already reads around them; and a product [m,1] x [1,n] - the
    // reference's way to broadcast a column or a row (core/ops/basic.d:370-381) - as the node
    // mul(per-row element, per-column element) of the chain's [m, n] view.
    auto outer_cols = [&](int id) -> size_t {   // n of such a product, else 0
        const Operation &o = g.ops[id];
        if (o.opType != "matmul" || o.deps.size() != 2 || o.rank() != 2 || o.dtype != DOPT_HIP_F32) return 0;
        const Operation &l = g.ops[o.deps[0]], &r = g.ops[o.deps[1]];
        if (l.rank() != 2 || r.rank() != 2 || l.shape[1] != 1 || r.shape[0] != 1) return 0;
        return o.shape[1];
    };
    // with one row or one column the product is a tensor times a single element: no [rows, inner] view needed
    auto outer_grid = [&](int id) -> size_t {
        const size_t n = outer_cols(id);
        return n > 1 && g.ops[id].shape[0] > 1 ? n : 0;
    };
    auto is_pw = [&](int id) {
        const Operation &o = g.ops[id];
        if (!live[id] || alias[id].source >= 0 || fusedKind[id] || o.dtype != DOPT_HIP_F32 || o.volume() == 0) return false;
        if (o.opType == "reluGrad" && o.deps.size() == 3) {
            for (const Use &u : uses[id])
                if (fusedKind[u.op] == 3 || fusedKind[u.op] == 8) return false;   // that batchNormGrad reads dy and y itself
            return true;
        }
        if (outer_cols(id)) return true;
        const int arity = dopt_hip_pointwise_arity(o.opType.c_str());
        return arity > 0 && arity == (int)o.deps.size();
    };
    std::vector<int> chainOf((size_t)nops, -1);              // the operation that ends the chain
    std::vector<std::vector<int>> chainOps((size_t)nops);    // per chain end: its members
    std::vector<size_t> chainInner((size_t)nops, 0);         // per chain end: columns of its [rows, inner] view, once a member needs one
    for (auto it = p->mOps.rbegin(); it != p->mOps.rend(); ++it) {
        const int id = *it;
        if (!is_pw(id)) continue;
        int target = -1;
        bool joins = !isOutput(id) && !uses[id].empty();
        auto reader_joins = [&](const Use &u, size_t volume) {   // the reader is a member of the one chain, and reads all of it
            if (chainOf[u.op] < 0 || u.off != 0 || g.ops[u.op].volume() != volume) joins = false;
            else if (g.ops[u.op].opType == "reluGrad" && u.slot == 1) joins = false;   // the y operand is not part of the node
            else if (target < 0) target = chainOf[u.op];
            else if (target != chainOf[u.op]) joins = false;
        };
        for (const Use &u : uses[id]) {
            if (!joins) break;
            // A one-element value that is only ever broadcast (repeat) into members of one chain - the scalar arithmetic
            // of a loss term or an update rule in front of the tensor it scales - is a node of that chain too: every
            // thread computes it again from the one-element operands, with the stand-alone kernel's expression.
            const Operation &ro = g.ops[u.op];
            if (g.ops[id].volume() == 1 && ro.opType == "repeat" && ro.deps.size() == 1 && u.off == 0 && u.slot == 0 &&
                ro.volume() > 1 && alias[u.op].source < 0 && !isOutput(u.op) && live[u.op] && !fusedKind[u.op] && !uses[u.op].empty()) {
                for (const Use &u2 : uses[u.op]) {
                    if (!joins) break;
                    reader_joins(u2, ro.volume());
                }
                continue;
            }
            // the same through the reference's other broadcast, the product with a ones vector ([n,1] x [1,1] or
            // [1,1] x [1,n], core/ops/basic.d:370-381): the member reads the value as its one-element operand
            if (g.ops[id].volume() == 1 && ro.volume() > 1 && outer_cols(u.op) && chainOf[u.op] >= 0 && u.off == 0 &&
                ((u.slot == 1 && ro.shape[1] == 1) || (u.slot == 0 && ro.shape[0] == 1))) {
                reader_joins(u, ro.volume());
                continue;
            }
            reader_joins(u, g.ops[id].volume());
        }
        if (joins && chainOps[target].size() >= 48) joins = false;
        const size_t cols = outer_grid(id);
        if (joins && cols && chainInner[target] && chainInner[target] != cols) joins = false;
        chainOf[id] = joins ? target : id;
        chainOps[chainOf[id]].push_back(id);
        if (cols) chainInner[chainOf[id]] = cols;
    }
    for (int end : p->mOps) {
        if (chainOf[end] != end || chainOps[end].size() < 2) continue;
        std::vector<int> members;                             // in execution order
        for (int id : p->mOps)
            if (chainOf[id] == end) members.push_back(id);
        std::vector<int> inputs;                              // operations whose buffers the kernel reads
        std::vector<unsigned char> kinds;                     // 0 tensor, 1 one element, 2 per row, 3 per column
        std::vector<int> nodeOf((size_t)nops, -1);
        struct Node { std::string op; int lhs, rhs; };
        std::vector<Node> nodes;
        auto input_index = [&](int op, int kind) {
            for (size_t k = 0; k < inputs.size(); k++)
                if (inputs[k] == op && kinds[k] == (unsigned char)kind) return (int)k;
            inputs.push_back(op);
            kinds.push_back((unsigned char)kind);
            return (int)inputs.size() - 1;
        };
        auto operand = [&](int dep) {                         // index of a member's operand: a node (<= -2) or an input
            size_t off;
            const int r = root(dep, &off);
            if (chainOf[r] == end && nodeOf[r] >= 0 && off == 0) return -2 - nodeOf[r];
            const Operation &ro = g.ops[r];
            size_t soff = 0;
            if (ro.opType == "repeat" && ro.deps.size() == 1 && off == 0 && alias[r].source < 0 &&
                g.ops[ro.deps[0]].volume() == 1 && g.ops[root(ro.deps[0], &soff)].dtype == DOPT_HIP_F32) {
                const int sr = root(ro.deps[0], &soff);
                if (chainOf[sr] == end && nodeOf[sr] >= 0 && soff == 0) return -2 - nodeOf[sr];   // a one-element member
                return input_index(ro.deps[0], 1);
            }
            // the operands of a one-element member of a larger chain are single elements
            if (g.ops[dep].volume() == 1 && g.ops[end].volume() > 1) return input_index(dep, 1);
            return input_index(dep, 0);
        };
        for (int id : members) {
            const Operation &o = g.ops[id];
            Node node{o.opType, -1, -1};
            if (outer_cols(id)) {
                node.op = "mul";
                const bool one_col = o.shape[1] == 1, one_row = o.shape[0] == 1;
                auto element = [&](int dep, int kind) {   // a single element may be a one-element member of this chain
                    size_t eoff;
                    const int sr = root(dep, &eoff);
                    if (kind == 1 && chainOf[sr] == end && nodeOf[sr] >= 0 && eoff == 0) return -2 - nodeOf[sr];
                    return input_index(dep, kind);
                };
                node.lhs = element(o.deps[0], one_row ? 1 : (one_col ? 0 : 2));
                node.rhs = element(o.deps[1], one_col ? 1 : (one_row ? 0 : 3));
            } else if (o.opType == "reluGrad") {
                node.lhs = operand(o.deps[0]);
                node.rhs = operand(o.deps[2]);
            } else {
                node.lhs = operand(o.deps[0]);
                if (o.deps.size() > 1) node.rhs = operand(o.deps[1]);
            }
            nodeOf[id] = (int)nodes.size();
            nodes.push_back(node);
        }
        if (inputs.empty() || inputs.size() > 12) continue;   // too wide: its members keep their own kernels
        const int nin = (int)inputs.size();
        for (Node &n : nodes) {
            if (n.lhs <= -2) n.lhs = nin + (-2 - n.lhs);
            if (n.rhs <= -2) n.rhs = nin + (-2 - n.rhs);
            if (n.rhs < 0) n.rhs = n.lhs;
        }
        for (int id : members) fusedKind[id] = 7;
        inputsOf[end] = inputs;
        const size_t count = g.ops[end].volume(), inner = chainInner[end];
        prebuilt[end] = make([=](const std::vector<const void *> &in, void *out) {
            const char *names[64];
            int lhs[64], rhs[64];
            for (size_t j = 0; j < nodes.size(); j++) {
                names[j] = nodes[j].op.c_str();
                lhs[j] = nodes[j].lhs;
                rhs[j] = nodes[j].rhs;
            }
            return dopt_hip_pointwise_chain(DOPT_HIP_F32, count, inner, nin, in.data(), kinds.data(), (int)nodes.size(),
                                            names, lhs, rhs, out);
        });
        prebuiltLabel[end] = "pointwise*" + std::to_string(nodes.size());   // no spaces: profile lines are split on them
    }
}

void HIPPlan::Builder::absorbBiasGrads()
{
    // addBiasGrad(dx of a batchNormGrad): the batch-norm kernel writes the bias gradient too.  The
    // addBiasGrad operation keeps its buffer but gets no kernel of its own.
    if (flags & DOPT_HIP_PLAN_FUSE) {
        for (int id : p->mOps) {
            const Operation &op = g.ops[id];
            if (op.opType != "addBiasGrad" || op.deps.size() != 1 || alias[id].source >= 0) continue;
            size_t off = 0;
            int r = op.deps[0];
            while (alias[r].source >= 0) {
                off += alias[r].offset;
                r = alias[r].source;
            }
            const Operation &bg = g.ops[r];
            if (bg.opType != "batchNormGrad" || bg.deps.size() != 3 || off != 0 || biasGradOf[r] >= 0) continue;
            const Operation &x = g.ops[bg.deps[1]];
            if (x.rank() < 2 || op.volume() != x.shape[1] || g.ops[op.deps[0]].volume() != x.volume()) continue;
            biasGradOf[r] = id;
            absorbed[id] = 1;
        }
    }
}

void HIPPlan::Builder::absorbPools()
{
    // maxpool [2, 2] of a batch norm's y part (through the relu that became an alias of it, or directly): the
    // batch-norm kernel has the values in registers and writes the pooled tensor too.  The maxpool operation
    // keeps its buffer but gets no kernel of its own.
    if (!(flags & DOPT_HIP_PLAN_FUSE)) return;
    for (int id : p->mOps) {
        const Operation &op = g.ops[id];
        if (op.opType != "maxpool" || op.deps.size() != 1 || alias[id].source >= 0 || op.dtype != DOPT_HIP_F32) continue;
        const auto *dims = sizes_attr(op, "dims");
        const auto &xs = g.ops[op.deps[0]].shape;
        if (!dims || dims->size() != 2 || (*dims)[0] != 2 || (*dims)[1] != 2 || xs.size() != 4 || xs[2] % 2 || xs[3] % 2) continue;
        size_t off;
        const int b = root(op.deps[0], &off);
        const Operation &bn = g.ops[b];
        if (bn.opType != "batchNormTrain" || bn.deps.size() != 5 || off != 0 || poolOf[b] >= 0 || prebuilt[b] ||
            (fusedKind[b] != 0 && fusedKind[b] != 2) || g.ops[bn.deps[0]].shape != xs || op.volume() == 0)
            continue;
        poolOf[b] = id;
        absorbed[id] = 1;
    }
}

void HIPPlan::Builder::markNeeded()
{
    // operations whose results are actually consumed (everything, unless rewrites created dead ones)
    {
        std::vector<int> work(outputs.begin(), outputs.end());
        while (!work.empty()) {
            int id = work.back();
            work.pop_back();
            if (needed[id]) continue;
            needed[id] = 1;
            if (alias[id].source >= 0) work.push_back(alias[id].source);
            else for (int d : inputsOf[id]) work.push_back(d);
        }
    }
}

int HIPPlan::Builder::prepackFilters()
{
    // Filters packed ahead (DOPT_HIP_PLAN_FUSE): the forward and backward-data kernels of 3x3
    // convolutions read the filter in their own layout.  When the filter is a variable or a constant
    // - fixed while the plan runs - every such layout of the plan is produced by ONE launch at the
    // start of each execution instead of one small launch in front of every convolution.
    if (flags & DOPT_HIP_PLAN_FUSE) {
        for (int id : p->mOps) {
            if (!needed[id] || alias[id].source >= 0 || absorbed[id] || prebuilt[id]) continue;
            const Operation &op = g.ops[id];
            Prepack k{};
            k.op = id;
            const Operation *cv = nullptr;
            if (fusedKind[id] == 1) cv = &g.ops[op.deps[0]];
            else if (!fusedKind[id] && op.opType == "convolution" && op.deps.size() == 2) cv = &op;
            if (cv) {
                const auto *pad = sizes_attr(*cv, "padding"), *stride = sizes_attr(*cv, "stride");
                const auto &x = g.ops[cv->deps[0]].shape, &w = g.ops[cv->deps[1]].shape;
                if (!pad || !stride || x.size() != 4 || w.size() != 4 || cv->dtype != DOPT_HIP_F32) continue;
                k.filter = cv->deps[1];
                k.d = conv_desc(x, w, *pad, *stride);
            } else if (!fusedKind[id] && op.opType == "convolutionFeaturesGrad" && op.deps.size() == 2) {
                const auto *pad = sizes_attr(op, "padding"), *stride = sizes_attr(op, "stride");
                const auto &w = g.ops[op.deps[1]].shape;
                if (!pad || !stride || op.shape.size() != 4 || w.size() != 4 || op.dtype != DOPT_HIP_F32) continue;
                k.filter = op.deps[1];
                k.bwd = 1;
                k.d = conv_desc(op.shape, w, *pad, *stride);
            } else {
                continue;
            }
            if (!is_leaf(g.ops[k.filter])) continue;
            const size_t bytes = dopt_hip_conv_packed_bytes(&k.d, k.bwd);
            if (bytes == 0) continue;
            // the forward and the backward-data convolution of a layer may read the very same copy
            const int layout = dopt_hip_conv_packed_layout(&k.d, k.bwd);
            for (const Prepack &other : packs)
                if (other.owner && other.filter == k.filter && memcmp(&other.d, &k.d, sizeof(k.d)) == 0 &&
                    dopt_hip_conv_packed_layout(&other.d, other.bwd) == layout)
                    k.buf = other.buf;
            if (layout == 3) k.buf = g.ops[k.filter].value;   // such kernels read the filter as it lies: nothing to pack (the
                                                              // step reads the filter operand of each run, see buildSteps)
            k.owner = k.buf == nullptr;
            k.late = layout == 2;
            if (k.owner) {
                if (int rc = dopt_hip_malloc(&k.buf, bytes)) return rc;
                p->mOwned.push_back(k.buf);
                p->mBufferBytes += bytes;
            }
            packOf[id] = (int)packs.size();
            packs.push_back(k);
        }
    }
    // The 3x3 layouts are small and many: one launch at the start of the run makes them all.  The
    // dense matrices of 2x2-image layers are 16 MB each and made by a launch of their own, so each is
    // made just before the convolution that reads it first and is still in the caches when it does.
    std::vector<Prepack> early;
    for (const Prepack &k : packs)
        if (k.owner && !k.late) early.push_back(k);
    if (!early.empty()) pushPackStep(early);
    return DOPT_HIP_OK;
}

// convolutionFeaturesGrad and convolutionFiltersGrad of one layer read the same dy and nothing of each other: where
// the former runs on a packed filter they become one step (dopt_hip_conv_bwd_pair_packed_open), placed where the
// earlier of the two stands in the order - checked below: every input of either is ready there - and every reader of
// either comes after its own, later or equal, position.
void HIPPlan::Builder::pairBackward()
{
    if (!(flags & DOPT_HIP_PLAN_FUSE)) return;
    std::vector<int> pos((size_t)nops, -1);
    for (size_t i = 0; i < p->mOps.size(); i++) pos[p->mOps[i]] = (int)i;
    std::vector<char> taken((size_t)nops, 0);
    for (int bd : p->mOps) {
        if (packOf[bd] < 0 || !needed[bd]) continue;
        const Prepack &pk = packs[(size_t)packOf[bd]];
        if (!pk.bwd || dopt_hip_conv_packed_layout(&pk.d, 1) != 1) continue;   // 3x3 patch layout only
        const Operation &bo = g.ops[bd];
        size_t dyoff;
        const int dyroot = root(bo.deps[0], &dyoff);
        const auto *pad = sizes_attr(bo, "padding"), *stride = sizes_attr(bo, "stride");
        for (int fg : p->mOps) {
            const Operation &fo = g.ops[fg];
            if (fo.opType != "convolutionFiltersGrad" || fo.deps.size() != 2 || !needed[fg] || taken[fg] || absorbed[fg] ||
                alias[fg].source >= 0 || prebuilt[fg] || fusedKind[fg] || fo.dtype != DOPT_HIP_F32)
                continue;
            size_t off2;
            if (root(fo.deps[0], &off2) != dyroot || off2 != dyoff) continue;
            const auto *pad2 = sizes_attr(fo, "padding"), *stride2 = sizes_attr(fo, "stride");
            if (!pad || !stride || !pad2 || !stride2 || *pad != *pad2 || *stride != *stride2) continue;
            if (fo.shape != g.ops[pk.filter].shape || g.ops[fo.deps[1]].shape != bo.shape) continue;
            const int first = pos[bd] < pos[fg] ? bd : fg, second = first == bd ? fg : bd;
            // The pair runs where `first` stands, so whatever else `second` reads (x of the filter gradient, a
            // computed filter) must have been made before that place; a graph written by hand may compute it in
            // between (gradient graphs never do: both read values of the forward pass).  Such a couple stays two steps.
            bool ready = true;
            for (int d : g.ops[second].deps) {
                size_t o;
                const int r = root(d, &o);
                if (!is_leaf(g.ops[r]) && pos[r] > pos[first]) ready = false;
            }
            if (!ready) continue;
            pairOf[bd] = fg;
            taken[fg] = 1;
            pairLead[first] = bd;
            pairLater[second] = 1;
            break;
        }
    }
}

void HIPPlan::Builder::pushPackStep(const std::vector<Prepack> &which)
{
    std::vector<dopt_hip_conv_desc> descs;
    std::vector<int> bwd;
    std::vector<float *> bufs;
    Step s;
    s.op = -1;
    s.label = "filterPack";
    for (const Prepack &k : which) {
        descs.push_back(k.d);
        bwd.push_back(k.bwd);
        bufs.push_back((float *)k.buf);
        s.inputOps.push_back(k.filter);
    }
    s.kernel = make([=](const std::vector<const void *> &in, void *) {
        return dopt_hip_conv_pack_batch((int)descs.size(), descs.data(), bwd.data(), (const float *const *)in.data(),
                                        bufs.data());
    });
    s.inputs.resize(s.inputOps.size());
    s.inputBytes.resize(s.inputOps.size());
    for (size_t i = 0; i < s.inputOps.size(); i++) s.inputBytes[i] = g.ops[s.inputOps[i]].bytes();
    p->mSteps.push_back(std::move(s));
}

int HIPPlan::Builder::allocateBuffers()
{
    // buffers first: a fused kernel may write into the buffer of a later operation
    for (int id : p->mOps) {
        if (!needed[id] || is_leaf(g.ops[id]) || alias[id].source >= 0) continue;
        void *buf = nullptr;
        if (int rc = dopt_hip_malloc(&buf, g.ops[id].bytes())) return rc;
        if (buf) p->mOwned.push_back(buf);
        p->mBufferBytes += g.ops[id].bytes();
        p->mResults[id] = buf;
    }
    return DOPT_HIP_OK;
}

// batchNormTrain (+ relu) whose kernel also fills the buffer of the maxpool behind it; `open`: its input is a
// convolution result that may arrive as partial copies (see openSplitSums).
std::unique_ptr<HIPKernel> HIPPlan::Builder::makePooledTrain(int id, std::shared_ptr<dopt_hip_split_sum> open, std::string *label)
{
    const Operation &op = g.ops[id];
    auto it = op.doubleAttrs.find("momentum");
    if (it == op.doubleAttrs.end()) {
        fail(DOPT_HIP_ERR_INVALID, "batchNormTrain has no 'momentum' attribute");
        return nullptr;
    }
    const double momentum = it->second;
    const auto &xs = g.ops[op.deps[0]].shape;
    const size_t N = xs[0], C = xs[1], H = xs[2], W = xs[3];
    const int relu = fusedKind[id] == 2;
    float *pooled = (float *)p->mResults[poolOf[id]];
    *label = std::string("batchNormTrain") + (relu ? "+relu" : "") + "+maxpool";
    return make([=](const std::vector<const void *> &in, void *out) {
        if (open && open->value != in[0]) return fail(DOPT_HIP_ERR_RUNTIME, "plan: open convolution result is not the batch norm's input");
        return dopt_hip_bn_train_pool(N, C, H, W, momentum, (const float *)in[0], open.get(), (const float *)in[1],
                                      (const float *)in[2], (const float *)in[3], (const float *)in[4], (float *)out, relu, pooled);
    });
}

int HIPPlan::Builder::buildSteps()
{
    // kernels and buffers
    for (int at : p->mOps) {
        if (!needed[at] || pairLater[at]) continue;
        const int id = pairLead[at] >= 0 ? pairLead[at] : at;   // a backward pair is built where its first operation stands
        const Operation &op = g.ops[id];
        if (is_leaf(op)) {
            if (!op.value && op.bytes() > 0)
                return fail(DOPT_HIP_ERR_INVALID, "%s %d has no value buffer", op.opType.c_str(), id);
            p->mResults[id] = op.value;
            continue;
        }
        if (alias[id].source >= 0) continue;  // resolved per execution
        if (absorbed[id]) continue;           // written by the batch-norm kernel it follows
        std::unique_ptr<HIPKernel> k;
        std::string label = op.opType;
        void *extra = biasGradOf[id] >= 0 && needed[biasGradOf[id]] ? p->mResults[biasGradOf[id]] : nullptr;
        std::vector<int> stepInputs = inputsOf[id];
        bool onPacked = false;
        if (packOf[id] >= 0) {  // the filter operand is read from its packed copy
            const Prepack pk = packs[(size_t)packOf[id]];
            if (pk.owner && pk.late) pushPackStep({pk});
            const float *packed = (const float *)pk.buf;
            const dopt_hip_conv_desc d = pk.d;
            onPacked = true;
            // layout 3: the kernel reads the filter itself, which is then one more input of the step (its last)
            const bool asIs = dopt_hip_conv_packed_layout(&d, pk.bwd) == 3;
            const int fi = !asIs ? -1 : pk.bwd ? 1 : fusedKind[id] == 1 ? 2 : 1;
            convSteps.push_back({0, id, pk.bwd, !pk.bwd && fusedKind[id] == 1, d, packed, fi});
            if (pk.bwd && pairOf[id] >= 0) {
                stepInputs = {op.deps[0], g.ops[pairOf[id]].deps[1]};
                float *dw = (float *)p->mResults[pairOf[id]];
                k = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_bwd_pair_packed_open(&d, (const float *)in[0], packed, (const float *)in[1], (float *)out,
                                                              dw, nullptr, nullptr);
                });
                label = "convolutionFeaturesGrad+convolutionFiltersGrad";
            } else if (pk.bwd) {
                stepInputs = {op.deps[0]};
                if (asIs) stepInputs.push_back(pk.filter);
                k = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_bwd_data_packed(&d, (const float *)in[0], fi >= 0 ? (const float *)in[fi] : packed,
                                                         (float *)out);
                });
            } else if (fusedKind[id] == 1) {
                stepInputs = {inputsOf[id][0], inputsOf[id][2]};
                if (asIs) stepInputs.push_back(pk.filter);
                k = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_fwd_bias_packed(&d, (const float *)in[0], fi >= 0 ? (const float *)in[fi] : packed,
                                                         (const float *)in[1], (float *)out);
                });
                label = "convolution+addBias";
            } else {
                stepInputs = {op.deps[0]};
                if (asIs) stepInputs.push_back(pk.filter);
                k = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_fwd_bias_packed(&d, (const float *)in[0], fi >= 0 ? (const float *)in[fi] : packed,
                                                         nullptr, (float *)out);
                });
            }
        } else if (prebuilt[id]) {
            k = std::move(prebuilt[id]);
            label = prebuiltLabel[id];
        } else if (poolOf[id] >= 0 && needed[poolOf[id]]) {
            k = makePooledTrain(id, nullptr, &label);
        } else if (fusedKind[id] || extra) {
            k = make_fused(g, id, fusedKind[id], extra, &label);
        } else {
            auto it = kernelCtrs().find(op.opType);
            if (it == kernelCtrs().end())
                return fail(DOPT_HIP_ERR_UNSUPPORTED, "Could not construct a HIP kernel for operation of type '%s'",
                            op.opType.c_str());
            clear_error();
            k = it->second(g, id);
        }
        if (!k) {
            std::string why = dopt_hip_last_error();
            return fail(DOPT_HIP_ERR_INVALID, "Could not construct a HIP kernel for operation of type '%s': %s",
                        op.opType.c_str(), why.empty() ? "constructor returned null" : why.c_str());
        }
        if (flags & DOPT_HIP_PLAN_TIMING_SHAPES) {
            label += "@";
            for (size_t i = 0; i < op.shape.size(); i++) label += (i ? "x" : "") + std::to_string(op.shape[i]);
        }
        Step s;
        s.op = id;
        s.label = label;
        s.inputOps = stepInputs;
        s.writes = tinyWrites[id];
        s.kernel = std::move(k);
        s.inputs.resize(s.inputOps.size());
        s.inputBytes.resize(s.inputOps.size());
        for (size_t i = 0; i < s.inputOps.size(); i++) s.inputBytes[i] = g.ops[s.inputOps[i]].bytes();
        p->mSteps.push_back(std::move(s));
        if (onPacked) convSteps.back().step = p->mSteps.size() - 1;
    }
    return DOPT_HIP_OK;
}

// Steps that nothing in the plan waits for - the weight and bias gradients of dense layers, the filter gradients of
// layers whose backward-data runs apart from them - are each a launch of a few microseconds, and between two launches
// of one queue the device idles about as long.  Those that read nothing but values made earlier and are read by nobody
// (their values only leave the plan) can run in any order and all at once: the plain products of the plan become one
// dopt_hip_sgemm_batch, the filter gradients of 2x2-image layers one dopt_hip_conv_bwd_filter_batch, each placed
// where the last of its members stood (everything they read is older than that, and nothing was going to read them
// before).  The members run the kernel bodies they would have run alone: no value changes (DOPT_HIP_PLAN_FUSE).
void HIPPlan::Builder::batchIndependent()
{
    if (!(flags & DOPT_HIP_PLAN_FUSE)) return;
    auto base_label = [](const std::string &l) { return l.substr(0, l.find('@')); };
    struct Product { size_t step; MatmulInfo mi; };
    struct Wgrad { size_t step; dopt_hip_conv_desc d; };
    std::vector<Product> products;
    std::vector<Wgrad> wgrads;
    for (size_t i = 0; i < p->mSteps.size(); i++) {
        const Step &st = p->mSteps[i];
        const int id = st.op;
        if (id < 0 || !uses[id].empty() || !dynamic_cast<FnKernel *>(st.kernel.get())) continue;
        if (biasGradOf[id] >= 0 || poolOf[id] >= 0 || pairOf[id] >= 0 || pairLead[id] >= 0 || pairLater[id] || packOf[id] >= 0) continue;
        const Operation &op = g.ops[id];
        const std::string label = base_label(st.label);
        MatmulInfo mi;
        if ((label == "matmul" || label == "matmul+transpose") && (fusedKind[id] == 0 || fusedKind[id] == 6) &&
            plainProduct(id, &mi, false) && st.inputOps.size() == 2 && st.inputOps[0] == mi.a && st.inputOps[1] == mi.b &&
            products.size() < 64) {
            products.push_back({i, mi});
        } else if (label == "convolutionFiltersGrad" && op.opType == "convolutionFiltersGrad" && fusedKind[id] == 0 &&
                   op.deps.size() == 2 && op.dtype == DOPT_HIP_F32 && st.inputOps == op.deps && wgrads.size() < 64) {
            const auto *pad = sizes_attr(op, "padding"), *stride = sizes_attr(op, "stride");
            const auto &x = g.ops[op.deps[1]].shape;
            if (!pad || !stride || x.size() != 4 || op.shape.size() != 4 || x[2] != 2 || x[3] != 2) continue;
            wgrads.push_back({i, conv_desc(x, op.shape, *pad, *stride)});
        }
    }
    std::vector<char> drop(p->mSteps.size(), 0);
    const bool shapes = (flags & DOPT_HIP_PLAN_TIMING_SHAPES) != 0;
    if (products.size() >= 2) {
        Step b;
        b.op = -1;
        b.label = "matmul*" + std::to_string(products.size()) + (shapes ? "@" : "");
        std::vector<int> tA, tB;
        std::vector<size_t> M, N, K;
        std::vector<float *> outs;
        for (const Product &c : products) {
            tA.push_back(c.mi.tA); tB.push_back(c.mi.tB);
            M.push_back(c.mi.M); N.push_back(c.mi.N); K.push_back(c.mi.K);
            b.inputOps.push_back(c.mi.a);
            b.inputOps.push_back(c.mi.b);
            outs.push_back((float *)p->mResults[p->mSteps[c.step].op]);
            drop[c.step] = 1;
        }
        const int n = (int)products.size();
        b.kernel = make([=](const std::vector<const void *> &in, void *) {
            std::vector<const float *> A((size_t)n), B((size_t)n);
            for (int j = 0; j < n; j++) {
                A[(size_t)j] = (const float *)in[(size_t)(2 * j)];
                B[(size_t)j] = (const float *)in[(size_t)(2 * j + 1)];
            }
            return dopt_hip_sgemm_batch(n, tA.data(), tB.data(), M.data(), N.data(), K.data(), A.data(), B.data(), outs.data());
        });
        b.inputs.resize(b.inputOps.size());
        b.inputBytes.resize(b.inputOps.size());
        for (size_t i = 0; i < b.inputOps.size(); i++) b.inputBytes[i] = g.ops[b.inputOps[i]].bytes();
        const size_t at = products.back().step;
        drop[at] = 0;
        p->mSteps[at] = std::move(b);
    }
    if (wgrads.size() >= 2) {
        Step b;
        b.op = -1;
        b.label = "convolutionFiltersGrad*" + std::to_string(wgrads.size()) + (shapes ? "@" : "");
        std::vector<dopt_hip_conv_desc> descs;
        std::vector<float *> outs;
        for (const Wgrad &c : wgrads) {
            descs.push_back(c.d);
            const Operation &op = g.ops[p->mSteps[c.step].op];
            b.inputOps.push_back(op.deps[0]);
            b.inputOps.push_back(op.deps[1]);
            outs.push_back((float *)p->mResults[p->mSteps[c.step].op]);
            drop[c.step] = 1;
        }
        const int n = (int)wgrads.size();
        b.kernel = make([=](const std::vector<const void *> &in, void *) {
            std::vector<const float *> dy((size_t)n), x((size_t)n);
            for (int j = 0; j < n; j++) {
                dy[(size_t)j] = (const float *)in[(size_t)(2 * j)];
                x[(size_t)j] = (const float *)in[(size_t)(2 * j + 1)];
            }
            return dopt_hip_conv_bwd_filter_batch(n, descs.data(), dy.data(), x.data(), outs.data());
        });
        b.inputs.resize(b.inputOps.size());
        b.inputBytes.resize(b.inputOps.size());
        for (size_t i = 0; i < b.inputOps.size(); i++) b.inputBytes[i] = g.ops[b.inputOps[i]].bytes();
        const size_t at = wgrads.back().step;
        drop[at] = 0;
        p->mSteps[at] = std::move(b);
    }
    // close the ranks; the convolution steps remembered for openSplitSums move with them
    std::vector<size_t> moved(p->mSteps.size(), 0);
    std::vector<Step> kept;
    for (size_t i = 0; i < p->mSteps.size(); i++) {
        moved[i] = kept.size();
        if (!drop[i]) kept.push_back(std::move(p->mSteps[i]));
    }
    p->mSteps = std::move(kept);
    for (ConvStep &cs : convSteps) cs.step = moved[cs.step];
}

// A convolution that splits its reduction normally ends with a pass that adds the partial copies.
// When the step right behind it is the batch norm (forward) or batch-norm gradient (backward) that
// reads the whole result anyway, the convolution leaves the result open and that step adds the
// copies while it loads them: one launch and one pass over the data less per such pair
// (DOPT_HIP_PLAN_FUSE).  The two steps share a description of the open result; whether a result is
// open at all is decided by the library at each run (it is not when the reduction was not split).
void HIPPlan::Builder::openSplitSums()
{
    if (!(flags & DOPT_HIP_PLAN_FUSE)) return;
    for (const ConvStep &cs : convSteps) {
        if (cs.step + 1 >= p->mSteps.size()) continue;
        Step &conv = p->mSteps[cs.step], &next = p->mSteps[cs.step + 1];
        const int b = next.op;
        if (b < 0 || prebuilt[b] || next.inputOps.empty()) continue;
        const Operation &bo = g.ops[b];
        size_t off;
        if (root(next.inputOps[0], &off) != cs.op || off != 0) continue;   // first operand: x (forward) or dy (gradient)
        auto open = std::make_shared<dopt_hip_split_sum>();
        const dopt_hip_conv_desc d = cs.d;
        const float *packed = cs.packed;
        const int fi = cs.filterIn;   // >= 0: the kernel reads the filter operand itself
        size_t N, C, inner;
        if (!cs.bwd && bo.opType == "batchNormTrain" && bo.deps.size() == 5 && next.inputOps.size() == 5 &&
            (fusedKind[b] == 0 || fusedKind[b] == 2)) {
            auto it = bo.doubleAttrs.find("momentum");
            if (it == bo.doubleAttrs.end()) continue;
            const double momentum = it->second;
            const int relu = fusedKind[b] == 2;
            nci(g.ops[bo.deps[0]].shape, &N, &C, &inner);
            const bool bias = cs.bias;
            conv.kernel = make([=](const std::vector<const void *> &in, void *out) {
                return dopt_hip_conv_fwd_bias_packed_open(&d, (const float *)in[0], fi >= 0 ? (const float *)in[fi] : packed,
                                                          bias ? (const float *)in[1] : nullptr, (float *)out, open.get());
            });
            if (poolOf[b] >= 0 && needed[poolOf[b]]) {
                std::string unused;
                next.kernel = makePooledTrain(b, open, &unused);
            } else {
                next.kernel = make([=](const std::vector<const void *> &in, void *out) {
                    if (open->value != in[0]) return fail(DOPT_HIP_ERR_RUNTIME, "plan: open convolution result is not the batch norm's input");
                    return dopt_hip_bn_train_open(N, C, inner, momentum, open.get(), (const float *)in[1], (const float *)in[2],
                                                  (const float *)in[3], (const float *)in[4], (float *)out, relu);
                });
            }
        } else if (cs.bwd && bo.opType == "batchNormGrad" && bo.deps.size() == 3 &&
                   (((fusedKind[b] == 3 || fusedKind[b] == 8) && next.inputOps.size() == 4) ||
                    (fusedKind[b] == 0 && next.inputOps.size() == 3))) {
            // kind 8: the gradient arrives through a 2 x 2 max-pool and a relu (inputs [dpooled, y, x, scale]); kind 3:
            // through a relu ([dy, y, x, scale]); kind 0: as it is ([dy, x, scale])
            const int kind = fusedKind[b];
            const bool has_y = kind != 0;
            void *extra = biasGradOf[b] >= 0 && needed[biasGradOf[b]] ? p->mResults[biasGradOf[b]] : nullptr;
            const auto &xs = g.ops[bo.deps[1]].shape;
            if (kind == 8 && xs.size() != 4) continue;
            nci(xs, &N, &C, &inner);
            const size_t H = kind == 8 ? xs[2] : inner, W = kind == 8 ? xs[3] : 1;
            const int keep = uses[cs.op].size() == 1 && !isOutput(cs.op) ? 0 : 1;   // does anything else read dy?
            // the filter gradient of a backward pair stays open as well: the gradient kernel's launch adds its copies
            auto side = std::make_shared<dopt_hip_split_sum>();
            if (pairOf[cs.op] >= 0) {
                float *dw = (float *)p->mResults[pairOf[cs.op]];
                conv.kernel = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_bwd_pair_packed_open(&d, (const float *)in[0], packed, (const float *)in[1], (float *)out,
                                                              dw, open.get(), side.get());
                });
            } else {
                conv.kernel = make([=](const std::vector<const void *> &in, void *out) {
                    return dopt_hip_conv_bwd_data_packed_open(&d, (const float *)in[0], fi >= 0 ? (const float *)in[fi] : packed,
                                                              (float *)out, open.get());
                });
            }
            next.kernel = make([=](const std::vector<const void *> &in, void *out) {
                if (open->value != in[0]) return fail(DOPT_HIP_ERR_RUNTIME, "plan: open convolution result is not the gradient's input");
                const float *y = has_y ? (const float *)in[1] : nullptr;
                const float *x = (const float *)in[has_y ? 2 : 1], *scale = (const float *)in[has_y ? 3 : 2];
                if (kind == 8)
                    return dopt_hip_bn_grad_side(N, C, H, W, nullptr, nullptr, keep, (const float *)in[0], open.get(), y, x, scale,
                                                 (float *)out, (float *)extra, side.get());
                return dopt_hip_bn_grad_side(N, C, H, W, nullptr, open.get(), keep, nullptr, nullptr, y, x, scale, (float *)out,
                                             (float *)extra, side.get());
            });
        }
    }
}

void HIPPlan::Builder::rememberAliases()
{
    // remember aliases for the per-execution resolve pass
    for (int id : p->mOps)
        if (needed[id] && alias[id].source >= 0) p->mResults[id] = nullptr;
    p->mAliasSource.assign((size_t)nops, -1);
    p->mAliasOffset.assign((size_t)nops, 0);
    for (int id : p->mOps)
        if (needed[id] && alias[id].source >= 0) {
            p->mAliasSource[id] = alias[id].source;
            p->mAliasOffset[id] = alias[id].offset;
        }
    p->mNeeded = needed;
}

int HIPPlan::Builder::assignQueues()
{
    if (flags & DOPT_HIP_PLAN_OVERLAP) {
        // A filter gradient feeds nothing of the backward chain: it, and every step that reads a
        // side-queue result, goes to the side queue.  Steps keep their order within each queue.
        std::vector<char> onSide((size_t)nops, 0);
        auto producer = [&](int id) {   // the operation whose kernel wrote the buffer `id` names
            while (alias[id].source >= 0) id = alias[id].source;
            return id;
        };
        int fences = 1;   // the final join
        for (Step &st : p->mSteps) {
            if (st.op < 0) continue;
            bool reads_side = false;
            for (int in : st.inputOps) reads_side = reads_side || onSide[producer(in)];
            const bool wgrad = g.ops[st.op].opType == "convolutionFiltersGrad";
            // a step with a second output (the absorbed bias gradient) stays on the main queue
            if ((wgrad || reads_side) && biasGradOf[st.op] < 0 && poolOf[st.op] < 0 && pairOf[st.op] < 0) {
                st.lane = 1;
                st.fenceBefore = true;
                onSide[st.op] = 1;
                for (int w : st.writes) onSide[w] = 1;
                p->mUsesSide = true;
                fences++;
            } else if (reads_side) {
                st.joinSide = true;
                fences++;
            }
        }
        if (p->mUsesSide) {
            p->mFences.resize((size_t)fences);
            for (hipEvent_t &ev : p->mFences) DOPT_HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        }
    }
    else if (flags & DOPT_HIP_PLAN_OVERLAP_LIGHT) {
        // Small steps off the main chain: a step whose value reaches only plan outputs (directly or
        // through other such steps) and that moves at most a few megabytes.  Each is moved up to
        // right behind the last step that produces one of its inputs and runs on the side queue.
        const size_t n = p->mSteps.size();
        auto producer = [&](int id) {
            while (alias[id].source >= 0) id = alias[id].source;
            return id;
        };
        std::vector<int> stepOf((size_t)nops, -1);   // which step writes an operation's buffer
        for (size_t i = 0; i < n; i++) {
            const int op = p->mSteps[i].op;
            if (op < 0) continue;
            stepOf[op] = (int)i;
            if (biasGradOf[op] >= 0) stepOf[biasGradOf[op]] = (int)i;
            if (poolOf[op] >= 0) stepOf[poolOf[op]] = (int)i;
            if (pairOf[op] >= 0) stepOf[pairOf[op]] = (int)i;
            for (int w : p->mSteps[i].writes) stepOf[w] = (int)i;
        }
        std::vector<std::vector<int>> readers(n), producers(n);
        for (size_t i = 0; i < n; i++)
            for (int in : p->mSteps[i].inputOps) {
                const int s = stepOf[producer(in)];
                if (s >= 0 && s != (int)i) {
                    readers[(size_t)s].push_back((int)i);
                    producers[i].push_back(s);
                }
            }
        const size_t kLightBytes = (size_t)4 << 20;
        std::vector<char> side(n, 0);
        for (size_t i = n; i-- > 0;) {   // readers come later in the order, so they are decided first
            const Step &st = p->mSteps[i];
            if (st.op < 0 || biasGradOf[st.op] >= 0 || producers[i].empty()) continue;
            // by label: a fused step carries the operation it ends in (convolution+addBias ends in an addBias), and a
            // convolution must stay behind the step that packs its filter
            const std::string &t = g.ops[st.op].opType;
            if (!st.writes.empty()) continue;   // a run of tiny operations: some member may feed the main chain
            if (st.label.find("convolution") != std::string::npos || st.label.find("batchNorm") != std::string::npos ||
                t.compare(0, 11, "convolution") == 0 || t.compare(0, 9, "batchNorm") == 0 || t == "uniform")
                continue;
            size_t bytes = g.ops[st.op].bytes();
            for (size_t b : st.inputBytes) bytes += b;
            bool off = bytes <= kLightBytes;
            for (int r : readers[i]) off = off && side[(size_t)r];
            side[i] = off;
        }
        // new order: a side step goes right behind the last of its producers in the new order (behind
        // that producer's batch norm if the two share an open convolution result, and behind side steps
        // already placed there); a producer that is a side step itself counts where it was placed
        std::vector<char> glued(n, 0);   // step i must stay right in front of step i + 1
        for (const ConvStep &cs : convSteps)
            if (cs.step + 1 < n) glued[cs.step] = 1;
        std::vector<std::vector<int>> behind(n);
        std::vector<int> anchorOf(n, -1);
        for (size_t i = 0; i < n; i++) {
            if (!side[i]) continue;
            int a = -1;
            for (int pr : producers[i]) {
                int at = side[(size_t)pr] ? anchorOf[(size_t)pr] : pr;
                // (the step behind a convolution stays with it only if it stays on the main queue itself: a relu
                // that moves to the side queue is no anchor - what is placed behind it would never be emitted)
                if (!side[(size_t)pr] && glued[(size_t)pr] && !side[(size_t)pr + 1]) at += 1;
                a = std::max(a, at);
            }
            anchorOf[i] = a;
            behind[(size_t)a].push_back((int)i);
        }
        std::vector<Step> ordered;
        ordered.reserve(n);
        int fences = 1;
        bool any = false;
        for (size_t i = 0; i < n; i++) {
            if (side[i]) continue;
            ordered.push_back(std::move(p->mSteps[i]));
            bool first = true;
            for (int j : behind[i]) {
                Step &st = p->mSteps[(size_t)j];
                st.lane = 1;
                st.fenceBefore = first;   // one wait covers the steps placed together
                if (first) fences++;
                first = false;
                any = true;
                ordered.push_back(std::move(st));
            }
        }
        if (ordered.size() != n) return fail(DOPT_HIP_ERR_RUNTIME, "plan: %zu of %zu steps placed on the two queues", ordered.size(), n);
        p->mSteps = std::move(ordered);
        if (any) {
            p->mUsesSide = true;
            p->mFences.resize((size_t)fences);
            for (hipEvent_t &ev : p->mFences) DOPT_HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        }
    }
    return DOPT_HIP_OK;
}

int HIPPlan::Builder::createEvents()
{
    // what a recorded graph cannot reproduce: per-kernel timing events, the second queue, and `uniform`,
    // whose kernel takes a call counter that changes with every execution
    p->mGraphOk = !(flags & DOPT_HIP_PLAN_TIMING) && !p->mUsesSide;
    for (const Step &st : p->mSteps) {
        if (st.op >= 0 && g.ops[st.op].opType == "uniform") p->mGraphOk = false;
        if (!st.kernel->replayable()) p->mGraphOk = false;
    }
    if (flags & DOPT_HIP_PLAN_TIMING) {
        p->mEvents.resize(p->mSteps.size());
        for (auto &ev : p->mEvents) {
            DOPT_HIP_CHECK(hipEventCreate(&ev.first));
            DOPT_HIP_CHECK(hipEventCreate(&ev.second));
        }
    }
    return DOPT_HIP_OK;
}

int HIPPlan::create(Graph *graph, const std::vector<int> &outputs, unsigned flags, std::unique_ptr<HIPPlan> *out)
{
    registerBuiltinKernels();
    if (!ensure_init()) return DOPT_HIP_ERR_RUNTIME;
    const Graph &g = *graph;
    const int nops = (int)g.ops.size();
    for (int o : outputs)
        if (o < 0 || o >= nops) return fail(DOPT_HIP_ERR_INVALID, "plan output %d is not an operation of the graph", o);

    std::unique_ptr<HIPPlan> p(new HIPPlan());
    p->mGraph = graph;
    p->mFlags = flags;
    p->mOutputs = outputs;
    std::vector<char> seen((size_t)nops, 0);
    for (int o : outputs) toposort(g, o, seen, p->mOps);

    Builder b(g, p.get(), outputs, flags);
    if (int rc = b.findAliases()) return rc;
    for (int id : p->mOps) b.inputsOf[id] = g.ops[id].deps;
    if (flags & DOPT_HIP_PLAN_FUSE) {
        b.countReaders();
        b.fusePairs();
        b.foldTransposes();
        b.fuseDenseLayers();
        b.fuseDenseBackward();
        b.formTinyRuns();
        b.fuseSquareSums();
        b.formChains();
        b.absorbBiasGrads();
        b.absorbPools();
    }
    b.markNeeded();
    if (flags & DOPT_HIP_PLAN_FUSE) {
        if (int rc = b.prepackFilters()) return rc;
        b.pairBackward();
    }
    if (int rc = b.allocateBuffers()) return rc;
    if (int rc = b.buildSteps()) return rc;
    b.batchIndependent();
    b.openSplitSums();
    b.rememberAliases();
    if (flags & (DOPT_HIP_PLAN_OVERLAP | DOPT_HIP_PLAN_OVERLAP_LIGHT))
        if (int rc = b.assignQueues()) return rc;
    if (int rc = b.createEvents()) return rc;
    if (const char *dump = std::getenv("DOPT_HIP_PLAN_DUMP")) {   // the steps as they will run: queue, label, operation, inputs
        if (dump[0] && dump[0] != '0')
            for (size_t i = 0; i < p->mSteps.size(); i++) {
                const Step &st = p->mSteps[i];
                std::fprintf(stderr, "plan step %3zu queue %d%s%s %-44s op %d <-", i, st.lane, st.fenceBefore ? " (waits)" : "",
                             st.joinSide ? " (joins)" : "", st.label.c_str(), st.op);
                for (int in : st.inputOps) std::fprintf(stderr, " %d", in);
                std::fprintf(stderr, "\n");
            }
    }
    // Resolve aliases once against the variables' own values so that result() is meaningful before
    // the first execution (an alias of a variable that is later passed as an argument moves with it).
    if (int rc = p->resolve(0, nullptr, nullptr, nullptr)) return rc;
    *out = std::move(p);
    return DOPT_HIP_OK;
}

HIPPlan::~HIPPlan() { cleanup(); }

void HIPPlan::cleanup()
{
    if (mClean) return;
    for (void *b : mOwned) dopt_hip_free(b);
    mOwned.clear();
    for (int t = 0; t < 2; t++) {
        for (auto &kv : mHostArgs[t]) {
            if (kv.second.dev) dopt_hip_free(kv.second.dev);
            if (kv.second.pinned) dopt_hip_host_free(kv.second.pinned);
        }
        mHostArgs[t].clear();
        if (mArgDone[t]) (void)hipEventDestroy(mArgDone[t]);
        mArgDone[t] = nullptr;
        mArgUsed[t] = false;
    }
    for (auto &ev : mEvents) {
        (void)hipEventDestroy(ev.first);
        (void)hipEventDestroy(ev.second);
    }
    mEvents.clear();
    for (hipEvent_t ev : mFences) (void)hipEventDestroy(ev);
    mFences.clear();
    for (CapturedRun &c : mRuns) {
        if (c.exec) (void)hipGraphExecDestroy(c.exec);
        if (c.graph) (void)hipGraphDestroy(c.graph);
    }
    mRuns.clear();
    mClean = true;
}

int HIPPlan::resolve(int nargs, const int *argOps, const void *const *argPtrs, const int *argOnHost)
{
    const Graph &g = *mGraph;
    // variables: argument buffer if given, else the variable's own value (package.d:367-401)
    for (int id : mOps)
        if (mNeeded[id] && is_leaf(g.ops[id])) mResults[id] = g.ops[id].value;
    int slot = -1;   // the pair of copies this execution's host arguments go through
    for (int a = 0; a < nargs; a++) {
        const int id = argOps[a];
        if (id < 0 || id >= (int)g.ops.size() || g.ops[id].opType != "variable")
            return fail(DOPT_HIP_ERR_INVALID,
                        "All assignments in args must be for Operations with an opType of 'variable'");
        if (!mNeeded[id]) continue;
        if (argOnHost && argOnHost[a]) {
            const size_t bytes = g.ops[id].bytes();
            if (slot < 0) {
                slot = mArgTurn;
                mArgTurn ^= 1;
                // the execution before last read this slot's device copies, and its uploads read the staging memory
                if (mArgUsed[slot]) DOPT_HIP_CHECK(hipEventSynchronize(mArgDone[slot]));
            }
            HostArg &h = mHostArgs[slot][id];
            if (!h.dev && bytes)
                if (int rc = dopt_hip_malloc(&h.dev, bytes)) return rc;
            if (!h.pinned && bytes)
                if (int rc = dopt_hip_host_alloc(&h.pinned, bytes)) return rc;
            if (bytes) {
                if (!argPtrs[a]) return fail(DOPT_HIP_ERR_INVALID, "Failed to set contents of HIP buffer: null pointer");
                std::memcpy(h.pinned, argPtrs[a], bytes);   // once per execution; the caller's array is free again
                if (int rc = dopt_hip_copy_h2d_beside(h.dev, h.pinned, bytes)) return rc;
            }
            mResults[id] = h.dev;
        } else {
            mResults[id] = const_cast<void *>(argPtrs[a]);
        }
    }
    if (slot >= 0) {
        if (int rc = dopt_hip_upload_join()) return rc;   // the kernels queued from here on wait for the uploads
        mArgPending = slot;
    }
    for (int id : mOps)
        if (mNeeded[id] && mAliasSource[id] >= 0)
            mResults[id] = (char *)mResults[mAliasSource[id]] + mAliasOffset[id];
    for (Step &s : mSteps)
        for (size_t i = 0; i < s.inputOps.size(); i++) s.inputs[i] = mResults[s.inputOps[i]];
    return DOPT_HIP_OK;
}

// The kernels of one execution, in order, on whatever the library's queues are; shared by the direct
// path and by graph capture.
int HIPPlan::enqueue(int nrets, void *const *rets)
{
    const bool timing = !mEvents.empty();
    size_t fence = 0;
    auto order = [&](int first, int then) -> int {   // work queued on `then` from here on follows all of `first` so far
        DOPT_HIP_CHECK(hipEventRecord(mFences[fence], lane_stream(first)));
        DOPT_HIP_CHECK(hipStreamWaitEvent(lane_stream(then), mFences[fence], 0));
        fence++;
        return DOPT_HIP_OK;
    };
    for (size_t i = 0; i < mSteps.size(); i++) {
        Step &s = mSteps[i];
        if (s.lane == 1 && s.fenceBefore) {
            if (int rc = order(0, 1)) return rc;   // its inputs come from main-queue steps before it
        } else if (s.joinSide) {
            if (int rc = order(1, 0)) return rc;
        }
        set_lane(s.lane);
        if (timing) DOPT_HIP_CHECK(hipEventRecord(mEvents[i].first, stream()));
        void *result = s.op >= 0 ? mResults[s.op] : nullptr;   // a step that serves other steps has no operation of its own
        const size_t resultBytes = s.op >= 0 ? mGraph->ops[s.op].bytes() : 0;
        const int rc = s.kernel->execute(s.inputs, s.inputBytes, result, resultBytes);
        if (!rc && timing) DOPT_HIP_CHECK(hipEventRecord(mEvents[i].second, stream()));
        set_lane(0);
        if (rc) return rc;
    }
    if (mUsesSide)
        if (int rc = order(1, 0)) return rc;       // the outputs, and whatever the caller queues next, see both queues' work
    if (timing) {
        DOPT_HIP_CHECK(hipStreamSynchronize(stream()));
        for (size_t i = 0; i < mSteps.size(); i++) {
            float ms = 0.0f;
            DOPT_HIP_CHECK(hipEventElapsedTime(&ms, mEvents[i].first, mEvents[i].second));
            auto &slot = profiler[mSteps[i].label];
            slot.first += (double)ms * 1000.0;
            slot.second += 1;
        }
    }
    // package.d:419-422: the outputs go to the caller's buffers
    mRetDst.clear();
    mRetSrc.clear();
    mRetBytes.clear();
    for (int i = 0; i < nrets; i++) {
        if (!rets[i]) continue;
        const int o = mOutputs[(size_t)i];
        mRetDst.push_back(rets[i]);
        mRetSrc.push_back(mResults[o]);
        mRetBytes.push_back(mGraph->ops[o].bytes());
    }
    return dopt_hip_copy_d2d_batch((int)mRetDst.size(), mRetDst.data(), mRetSrc.data(), mRetBytes.data());
}

int HIPPlan::execute(int nargs, const int *argOps, const void *const *argPtrs, const int *argOnHost, int nrets,
                     void *const *rets)
{
    if (mClean) return fail(DOPT_HIP_ERR_INVALID, "plan was cleaned up");
    if (nrets > (int)mOutputs.size()) return fail(DOPT_HIP_ERR_INVALID, "more return buffers than plan outputs");

    // DOPT_HIP_PLAN_GRAPH: an execution is identified by the device pointers it binds (arguments and
    // return buffers).  The first execution with a given binding runs directly (run-time compilation,
    // workspace growth and pool allocations all happen there), the second is recorded into a HIP
    // graph while it runs, later ones replay that graph with one launch.
    bool graphable = mGraphOk && (mFlags & DOPT_HIP_PLAN_GRAPH);
    for (int a = 0; a < nargs && graphable; a++) graphable = !argOnHost[a];   // a host argument is uploaded anew every time
    if (graphable) {
        std::vector<const void *> key;
        for (int a = 0; a < nargs; a++) {
            key.push_back((const void *)(intptr_t)argOps[a]);
            key.push_back(argPtrs[a]);
        }
        key.push_back(nullptr);
        for (int i = 0; i < nrets; i++) key.push_back(rets[i]);
        CapturedRun *run = nullptr;
        for (CapturedRun &c : mRuns)
            if (c.key == key) run = &c;
        if (run && run->exec && run->wsGeneration != workspace_generation()) {
            // the workspace moved since this run was recorded (some other plan or call needed a larger
            // one): the recording holds the old address and must not be launched again; record anew
            (void)hipGraphExecDestroy(run->exec);
            if (run->graph) (void)hipGraphDestroy(run->graph);
            run->exec = nullptr;
            run->graph = nullptr;
        }
        if (run && run->exec) {
            mReplays++;
            DOPT_HIP_CHECK(hipGraphLaunch(run->exec, stream()));
            if (run->clusterKernels) bn_cluster_mark_unchecked();   // the next synchronisation point reads their error word
            return DOPT_HIP_OK;
        }
        if (!run) {
            if (mRuns.size() >= 8) {   // bindings keep changing: drop the oldest recording
                if (mRuns.front().exec) (void)hipGraphExecDestroy(mRuns.front().exec);
                if (mRuns.front().graph) (void)hipGraphDestroy(mRuns.front().graph);
                mRuns.erase(mRuns.begin());
            }
            mRuns.push_back(CapturedRun{key, nullptr, nullptr, 0, false});
        } else {
            if (int rc = resolve(nargs, argOps, argPtrs, argOnHost)) return rc;
            DOPT_HIP_CHECK(hipStreamBeginCapture(stream(), hipStreamCaptureModeRelaxed));
            set_capturing(true);
            const unsigned long clusterBefore = bn_cluster_launches();
            const int rc = enqueue(nrets, rets);
            run->clusterKernels = bn_cluster_launches() != clusterBefore;
            set_capturing(false);
            run->wsGeneration = workspace_generation();   // cannot change while recording: growth is refused
            hipGraph_t graph = nullptr;
            const hipError_t ended = hipStreamEndCapture(stream(), &graph);
            if (rc == DOPT_HIP_OK && ended == hipSuccess && graph &&
                hipGraphInstantiate(&run->exec, graph, nullptr, nullptr, 0) == hipSuccess) {
                run->graph = graph;
                DOPT_HIP_CHECK(hipGraphLaunch(run->exec, stream()));
                if (run->clusterKernels) bn_cluster_mark_unchecked();
                return DOPT_HIP_OK;
            }
            // something in this plan cannot be recorded (an allocation, a fill): nothing ran, run it directly from now on
            (void)hipGetLastError();
            if (graph) (void)hipGraphDestroy(graph);
            run->exec = nullptr;
            mGraphOk = false;
            clear_error();
        }
    }
    if (int rc = resolve(nargs, argOps, argPtrs, argOnHost)) return rc;
    const int rc = enqueue(nrets, rets);
    if (mArgPending >= 0) {   // behind everything that reads this execution's host arguments
        const int slot = mArgPending;
        mArgPending = -1;
        if (!mArgDone[slot]) DOPT_HIP_CHECK(hipEventCreateWithFlags(&mArgDone[slot], hipEventDisableTiming));
        DOPT_HIP_CHECK(hipEventRecord(mArgDone[slot], lane_stream(0)));
        mArgUsed[slot] = true;
    }
    return rc;
}

int HIPPlan::result(int op, void **ptr, size_t *bytes) const
{
    auto it = mResults.find(op);
    if (it == mResults.end()) return fail(DOPT_HIP_ERR_INVALID, "operation %d is not part of this plan", op);
    if (ptr) *ptr = it->second;
    if (bytes) *bytes = mGraph->ops[op].bytes();
    return DOPT_HIP_OK;
}

std::string HIPPlan::profile()
{
    std::string s;
    char line[256];
    for (auto &kv : profiler) {
        snprintf(line, sizeof(line), "%s %.1f %zu\n", kv.first.c_str(), kv.second.first, kv.second.second);
        s += line;
    }
    return s;
}

}  // namespace dopt

// ------------------------------------------------------------------------------- C ABI

using namespace dopt;

namespace {

int copy_text(const std::string &s, char *buf, size_t buf_bytes, size_t *needed)
{
    if (needed) *needed = s.size() + 1;
    if (buf && buf_bytes > 0) {
        size_t n = s.size() < buf_bytes - 1 ? s.size() : buf_bytes - 1;
        memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
    return DOPT_HIP_OK;
}

class CKernel : public HIPKernel {
public:
    explicit CKernel(dopt_hip_kernel k) : mK(k) {}
    ~CKernel() override
    {
        if (mK.destroy) mK.destroy(mK.self);
    }
    int execute(const std::vector<const void *> &inputs, const std::vector<size_t> &inputBytes, void *output,
                size_t outputBytes) override
    {
        return mK.execute(mK.self, (int)inputs.size(), inputs.data(), inputBytes.data(), output, outputBytes);
    }
    bool replayable() const override { return false; }   // the callback's host code would not run on a replay

private:
    dopt_hip_kernel mK;
};

bool valid_op(Graph *g, int op) { return g && op >= 0 && op < (int)g->ops.size(); }

}  // namespace

extern "C" {

int dopt_hip_graph_create(void **graph)
{
    DOPT_REQUIRE(graph != nullptr, "dopt_hip_graph_create: graph is null");
    *graph = new Graph();
    return DOPT_HIP_OK;
}

int dopt_hip_graph_destroy(void *graph)
{
    delete (Graph *)graph;
    return DOPT_HIP_OK;
}

int dopt_hip_graph_add_op(void *graph, const char *op_type, int dtype, int rank, const size_t *shape, int ndeps,
                          const int *deps, int *op_id)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(g && op_type && op_id, "dopt_hip_graph_add_op: null argument");
    DOPT_REQUIRE(rank >= 0 && rank <= 8 && (rank == 0 || shape), "dopt_hip_graph_add_op: rank must be 0..8");
    DOPT_REQUIRE(ndeps >= 0 && (ndeps == 0 || deps), "dopt_hip_graph_add_op: bad dependency list");
    if (dtype != DOPT_HIP_F32 && dtype != DOPT_HIP_I32)
        return fail(DOPT_HIP_ERR_UNSUPPORTED, "Element type not supported.");
    Operation op;
    op.opType = op_type;
    op.dtype = dtype;
    op.shape.assign(shape, shape + rank);
    for (int i = 0; i < ndeps; i++) {
        DOPT_REQUIRE(deps[i] >= 0 && deps[i] < (int)g->ops.size(), "dopt_hip_graph_add_op: dependency %d does not exist",
                     deps[i]);
        op.deps.push_back(deps[i]);
    }
    if (is_leaf(op)) {
        DOPT_REQUIRE(ndeps == 0, "%s takes no dependencies", op_type);
        if (int rc = dopt_hip_malloc(&op.value, op.bytes())) return rc;  // defaultVarAllocator
    }
    g->ops.push_back(std::move(op));
    *op_id = (int)g->ops.size() - 1;
    return DOPT_HIP_OK;
}

int dopt_hip_graph_set_attr_sizes(void *graph, int op, const char *key, const size_t *values, int n)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(valid_op(g, op) && key && n >= 0 && (n == 0 || values), "dopt_hip_graph_set_attr_sizes: bad argument");
    g->ops[op].sizeAttrs[key].assign(values, values + n);
    return DOPT_HIP_OK;
}

int dopt_hip_graph_set_attr_double(void *graph, int op, const char *key, double value)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(valid_op(g, op) && key, "dopt_hip_graph_set_attr_double: bad argument");
    g->ops[op].doubleAttrs[key] = value;
    return DOPT_HIP_OK;
}

int dopt_hip_graph_value(void *graph, int op, void **device_ptr, size_t *bytes)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(valid_op(g, op), "dopt_hip_graph_value: no such operation");
    DOPT_REQUIRE(is_leaf(g->ops[op]), "dopt_hip_graph_value: only variables and constants have a value");
    if (device_ptr) *device_ptr = g->ops[op].value;
    if (bytes) *bytes = g->ops[op].bytes();
    return DOPT_HIP_OK;
}

int dopt_hip_graph_op_type(void *graph, int op, const char **op_type, int *dtype, int *rank, size_t *shape8, int *ndeps)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(valid_op(g, op), "dopt_hip_graph_op_type: no such operation");
    const Operation &o = g->ops[op];
    if (op_type) *op_type = o.opType.c_str();
    if (dtype) *dtype = o.dtype;
    if (rank) *rank = (int)o.rank();
    if (shape8)
        for (size_t i = 0; i < o.rank() && i < 8; i++) shape8[i] = o.shape[i];
    if (ndeps) *ndeps = (int)o.deps.size();
    return DOPT_HIP_OK;
}

int dopt_hip_graph_op_dep(void *graph, int op, int index, int *dep)
{
    Graph *g = (Graph *)graph;
    DOPT_REQUIRE(valid_op(g, op) && dep && index >= 0 && index < (int)g->ops[op].deps.size(),
                 "dopt_hip_graph_op_dep: bad argument");
    *dep = g->ops[op].deps[(size_t)index];
    return DOPT_HIP_OK;
}

int dopt_hip_register_kernel(const char *op_name, dopt_hip_kernel_ctor ctor, void *user)
{
    DOPT_REQUIRE(op_name && ctor, "dopt_hip_register_kernel: null argument");
    return registerHIPKernel(op_name, [ctor, user](const Graph &g, int op) -> std::unique_ptr<HIPKernel> {
        dopt_hip_kernel k{};
        if (ctor((void *)&g, op, user, &k) != 0 || !k.execute) {
            if (!*dopt_hip_last_error()) fail(DOPT_HIP_ERR_INVALID, "kernel constructor refused the operation");
            return nullptr;
        }
        return std::unique_ptr<HIPKernel>(new CKernel(k));
    });
}

int dopt_hip_deregister_kernel(const char *op_name)
{
    DOPT_REQUIRE(op_name != nullptr, "dopt_hip_deregister_kernel: null argument");
    deregisterHIPKernel(op_name);
    return DOPT_HIP_OK;
}

int dopt_hip_list_operations(char *buf, size_t buf_bytes, size_t *needed)
{
    std::string s;
    for (const std::string &n : listHIPOperations()) s += n + "\n";
    return copy_text(s, buf, buf_bytes, needed);
}

int dopt_hip_plan_create(void *graph, int noutputs, const int *outputs, unsigned flags, void **plan)
{
    DOPT_REQUIRE(graph && plan && noutputs >= 0 && (noutputs == 0 || outputs), "dopt_hip_plan_create: bad argument");
    *plan = nullptr;
    std::unique_ptr<HIPPlan> p;
    if (int rc = HIPPlan::create((Graph *)graph, std::vector<int>(outputs, outputs + noutputs), flags, &p)) return rc;
    *plan = p.release();
    return DOPT_HIP_OK;
}

int dopt_hip_plan_execute(void *plan, int nargs, const int *arg_ops, const void *const *arg_ptrs, const int *arg_on_host,
                          int nrets, void *const *rets)
{
    DOPT_REQUIRE(plan != nullptr, "dopt_hip_plan_execute: plan is null");
    DOPT_REQUIRE(nargs >= 0 && (nargs == 0 || (arg_ops && arg_ptrs)) && nrets >= 0 && (nrets == 0 || rets),
                 "dopt_hip_plan_execute: bad argument");
    return ((HIPPlan *)plan)->execute(nargs, arg_ops, arg_ptrs, arg_on_host, nrets, rets);
}

int dopt_hip_plan_result(void *plan, int op, void **device_ptr, size_t *bytes)
{
    DOPT_REQUIRE(plan != nullptr, "dopt_hip_plan_result: plan is null");
    return ((HIPPlan *)plan)->result(op, device_ptr, bytes);
}

int dopt_hip_plan_stats(void *plan, size_t *kernels, size_t *buffer_bytes)
{
    DOPT_REQUIRE(plan != nullptr, "dopt_hip_plan_stats: plan is null");
    if (kernels) *kernels = ((HIPPlan *)plan)->kernelCount();
    if (buffer_bytes) *buffer_bytes = ((HIPPlan *)plan)->bufferBytes();
    return DOPT_HIP_OK;
}

int dopt_hip_plan_recordings(void *plan, size_t *recorded, size_t *replays)
{
    DOPT_REQUIRE(plan != nullptr, "dopt_hip_plan_recordings: plan is null");
    ((HIPPlan *)plan)->recordings(recorded, replays);
    return DOPT_HIP_OK;
}

int dopt_hip_plan_profile(void *plan, char *buf, size_t buf_bytes, size_t *needed)
{
    DOPT_REQUIRE(plan != nullptr, "dopt_hip_plan_profile: plan is null");
    return copy_text(((HIPPlan *)plan)->profile(), buf, buf_bytes, needed);
}

int dopt_hip_plan_destroy(void *plan)
{
    delete (HIPPlan *)plan;
    return DOPT_HIP_OK;
}

}  // extern "C"
