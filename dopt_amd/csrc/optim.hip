// Fused multi-tensor SGD / ADAM / AMSGrad updates.
//
// The reference has no optimizer kernels: online/source/dopt/online/{sgd,adam,amsgrad}.d build
// each rule as a graph of pointwise ops whose scalars are broadcast through GEMMs against a ones
// vector, roughly a dozen launches per parameter tensor per step.  Here every tensor of the
// model is updated in place by ONE launch.  Each graph node keeps its own fp32 rounding (this
// file is compiled without FMA contraction and with correctly rounded divide / sqrt), so the
// result is bit-identical to evaluating the un-fused graph.
#include <cmath>
#include <vector>

#include "common.h"

namespace {

using namespace dopt;

constexpr int kBlock = 256;
constexpr int kVecPerThread = 4;                         // float4 per lane per chunk
constexpr size_t kChunk = (size_t)kBlock * kVecPerThread * 4;  // 4096 elements per block-iteration

struct TensorDev {
    float *w;
    const float *g;
    float *m;
    float *v;
    float *vhat;
    size_t n;
    int skip_w;
    int vec;  // all pointers 16-byte aligned
};

struct ChunkDev {
    unsigned tensor;
    unsigned pad;
    size_t offset;  // first element of the chunk
};

struct Handle {
    int ntensors = 0;
    size_t nchunks = 0;
    bool has_v = true, has_vhat = true;
    TensorDev *tensors = nullptr;  // device
    ChunkDev *chunks = nullptr;    // device
};

enum Rule { kSgd = 0, kSgdNesterov = 1, kAdam = 2, kAmsgrad = 3 };

struct Scalars {
    float lr, mu;                    // sgd
    float eta, beta1, beta2, c1, c2, eps;  // adam / amsgrad
};

template <int kRule>
__device__ inline void update1(const Scalars &s, float &w, float g, float &m, float &v, float &vhat)
{
    if (kRule == kSgd) {
        float a = m * s.mu;          // x[1] * momentumRate            (sgd.d:59)
        float b = s.lr * g;          // learningRate * x[0]
        float nm = a + b;
        m = nm;
        w = w - nm;                  // sgd.d:63
    } else if (kRule == kSgdNesterov) {
        float a = m * s.mu;
        float b = s.lr * g;
        float nm = a - b;            // sgd.d:48
        float t0 = s.mu * nm;        // momentumRate * x[1]            (sgd.d:52)
        float t1 = w + t0;
        float t2 = s.lr * g;
        m = nm;
        w = t1 - t2;
    } else {
        if (kRule == kAmsgrad) vhat = vhat < v ? v : vhat;  // max(vhat, OLD v)   (amsgrad.d:63-66)
        float t0 = s.beta1 * m;
        float t1 = s.c1 * g;
        float nm = t0 + t1;          // adam.d:54
        float t2 = s.beta2 * v;
        float t3 = s.c2 * g;
        float t4 = t3 * g;           // ((1 - beta2) * g) * g
        float nv = t2 + t4;          // adam.d:59
        float sq = sqrtf(nv);
        float den = sq + s.eps;
        float q = nm / den;
        float step = s.eta * q;
        m = nm;
        v = nv;
        w = w - step;                // adam.d:63 -- AMSGrad uses v' here too (amsgrad.d:68-69)
    }
}

template <int kRule>
__global__ __launch_bounds__(kBlock) void optim_k(const TensorDev *tensors, const ChunkDev *chunks, size_t nchunks,
                                                   Scalars s)
{
    constexpr bool kHasV = kRule >= kAdam;
    constexpr bool kHasVhat = kRule == kAmsgrad;
    for (size_t ci = blockIdx.x; ci < nchunks; ci += gridDim.x) {
        const ChunkDev ch = chunks[ci];
        const TensorDev t = tensors[ch.tensor];
        const size_t begin = ch.offset;
        const size_t end = begin + kChunk < t.n ? begin + kChunk : t.n;
        if (t.vec && end - begin == kChunk) {
            float4 w[kVecPerThread], g[kVecPerThread], m[kVecPerThread], v[kVecPerThread], vh[kVecPerThread];
            const size_t b4 = begin >> 2;
#pragma unroll
            for (int u = 0; u < kVecPerThread; u++) {
                size_t i = b4 + (size_t)u * kBlock + threadIdx.x;
                w[u] = ((const float4 *)t.w)[i];
                g[u] = ((const float4 *)t.g)[i];
                m[u] = ((const float4 *)t.m)[i];
                if (kHasV) v[u] = ((const float4 *)t.v)[i];
                if (kHasVhat) vh[u] = ((const float4 *)t.vhat)[i];
            }
#pragma unroll
            for (int u = 0; u < kVecPerThread; u++) {
                size_t i = b4 + (size_t)u * kBlock + threadIdx.x;
                update1<kRule>(s, w[u].x, g[u].x, m[u].x, v[u].x, vh[u].x);
                update1<kRule>(s, w[u].y, g[u].y, m[u].y, v[u].y, vh[u].y);
                update1<kRule>(s, w[u].z, g[u].z, m[u].z, v[u].z, vh[u].z);
                update1<kRule>(s, w[u].w, g[u].w, m[u].w, v[u].w, vh[u].w);
                if (!t.skip_w) ((float4 *)t.w)[i] = w[u];
                ((float4 *)t.m)[i] = m[u];
                if (kHasV) ((float4 *)t.v)[i] = v[u];
                if (kHasVhat) ((float4 *)t.vhat)[i] = vh[u];
            }
        } else {
            for (size_t i = begin + threadIdx.x; i < end; i += kBlock) {
                float w = t.w[i], g = t.g[i], m = t.m[i];
                float v = kHasV ? t.v[i] : 0.0f, vh = kHasVhat ? t.vhat[i] : 0.0f;
                update1<kRule>(s, w, g, m, v, vh);
                if (!t.skip_w) t.w[i] = w;
                t.m[i] = m;
                if (kHasV) t.v[i] = v;
                if (kHasVhat) t.vhat[i] = vh;
            }
        }
    }
}

template <int kRule>
int launch(Handle *h, const Scalars &s)
{
    if (h->nchunks == 0) return DOPT_HIP_OK;
    size_t cap = (size_t)num_cus() * 16;
    unsigned grid = (unsigned)(h->nchunks < cap ? h->nchunks : cap);
    hipLaunchKernelGGL(optim_k<kRule>, dim3(grid), dim3(kBlock), 0, stream(), h->tensors, h->chunks, h->nchunks, s);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// The scalar prologue of online/adam.d:46-50, evaluated on the host in fp32, one rounding per
// node: nb = b * beta;  eta = (alpha * sqrt(1 - nb2)) / (1 - nb1).
void adam_scalars(float alpha, float beta1, float beta2, float eps, float *b1, float *b2, Scalars *s)
{
    volatile float nb1 = *b1 * beta1;
    volatile float nb2 = *b2 * beta2;
    volatile float one_m_nb2 = 1.0f - nb2;
    volatile float sq = sqrtf(one_m_nb2);
    volatile float num = alpha * sq;
    volatile float den = 1.0f - nb1;
    volatile float eta = num / den;
    volatile float c1 = 1.0f - beta1;
    volatile float c2 = 1.0f - beta2;
    *b1 = nb1;
    *b2 = nb2;
    s->eta = eta;
    s->beta1 = beta1;
    s->beta2 = beta2;
    s->c1 = c1;
    s->c2 = c2;
    s->eps = eps;
    s->lr = s->mu = 0.0f;
}

}  // namespace

extern "C" {

int dopt_hip_optim_create(int ntensors, const dopt_hip_tensor_ref *refs, void **handle)
{
    DOPT_REQUIRE(handle != nullptr, "dopt_hip_optim_create: handle is null");
    *handle = nullptr;
    DOPT_REQUIRE(ntensors >= 0 && (ntensors == 0 || refs), "dopt_hip_optim_create: bad tensor list");
    DOPT_ENSURE_INIT();
    Handle *h = new Handle();
    h->ntensors = ntensors;
    std::vector<TensorDev> tens((size_t)ntensors);
    std::vector<ChunkDev> chunks;
    for (int t = 0; t < ntensors; t++) {
        const dopt_hip_tensor_ref &r = refs[t];
        if (r.n > 0 && !(r.w && r.g && r.m)) {
            delete h;
            return fail(DOPT_HIP_ERR_INVALID, "dopt_hip_optim_create: tensor %d has a null w, g or m", t);
        }
        if (!r.v) h->has_v = false;
        if (!r.vhat) h->has_vhat = false;
        TensorDev &d = tens[(size_t)t];
        d.w = r.w;
        d.g = r.g;
        d.m = r.m;
        d.v = r.v;
        d.vhat = r.vhat;
        d.n = r.n;
        d.skip_w = r.skip_w;
        d.vec = aligned16(r.w) && aligned16(r.g) && aligned16(r.m) && (!r.v || aligned16(r.v)) &&
                (!r.vhat || aligned16(r.vhat));
        for (size_t off = 0; off < r.n; off += kChunk) chunks.push_back(ChunkDev{(unsigned)t, 0u, off});
    }
    h->nchunks = chunks.size();
    int rc = DOPT_HIP_OK;
    if (ntensors > 0) {
        rc = dopt_hip_malloc((void **)&h->tensors, tens.size() * sizeof(TensorDev));
        if (!rc) rc = dopt_hip_copy_h2d(h->tensors, tens.data(), tens.size() * sizeof(TensorDev));
    }
    if (!rc && !chunks.empty()) {
        rc = dopt_hip_malloc((void **)&h->chunks, chunks.size() * sizeof(ChunkDev));
        if (!rc) rc = dopt_hip_copy_h2d(h->chunks, chunks.data(), chunks.size() * sizeof(ChunkDev));
    }
    if (rc) {
        dopt_hip_free(h->tensors);
        dopt_hip_free(h->chunks);
        delete h;
        return rc;
    }
    *handle = h;
    return DOPT_HIP_OK;
}

int dopt_hip_optim_destroy(void *handle)
{
    if (!handle) return DOPT_HIP_OK;
    Handle *h = (Handle *)handle;
    dopt_hip_free(h->tensors);
    dopt_hip_free(h->chunks);
    delete h;
    return DOPT_HIP_OK;
}

int dopt_hip_sgd_step(void *handle, float lr, float mu, int nesterov)
{
    DOPT_REQUIRE(handle != nullptr, "dopt_hip_sgd_step: handle is null");
    Handle *h = (Handle *)handle;
    Scalars s{};
    s.lr = lr;
    s.mu = mu;
    return nesterov ? launch<kSgdNesterov>(h, s) : launch<kSgd>(h, s);
}

int dopt_hip_adam_step(void *handle, float alpha, float beta1, float beta2, float eps, float *b1, float *b2)
{
    DOPT_REQUIRE(handle && b1 && b2, "dopt_hip_adam_step: null argument");
    Handle *h = (Handle *)handle;
    DOPT_REQUIRE(h->has_v, "dopt_hip_adam_step: every tensor needs a second-moment buffer v");
    Scalars s{};
    adam_scalars(alpha, beta1, beta2, eps, b1, b2, &s);
    return launch<kAdam>(h, s);
}

int dopt_hip_amsgrad_step(void *handle, float alpha, float beta1, float beta2, float eps, float *b1, float *b2)
{
    DOPT_REQUIRE(handle && b1 && b2, "dopt_hip_amsgrad_step: null argument");
    Handle *h = (Handle *)handle;
    DOPT_REQUIRE(h->has_v && h->has_vhat, "dopt_hip_amsgrad_step: every tensor needs v and vhat buffers");
    Scalars s{};
    adam_scalars(alpha, beta1, beta2, eps, b1, b2, &s);
    return launch<kAmsgrad>(h, s);
}

}  // extern "C"
