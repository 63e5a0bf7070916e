// Spatial batch normalisation: training forward, backward and inference.
// Replaces cudnnBatchNormalizationForwardTraining / Backward / ForwardInference as called at
// cuda/source/dopt/cuda/nnet/cudnn7.d:608-610, :632-634, :650-652, including the reference's
// packed output layouts (core/source/dopt/core/ops/nnet.d:222-235).
//
// Channels of up to 32768 values take the channel-resident path (one launch, one read of the
// inputs; see bn_resident_k).  Larger channels take three launches, all deterministic (no atomics):
//   1. partial: block (channel, slice) accumulates shifted moments of its share of the channel
//      (shift K = first element of the channel, so that E[(x-K)^2] - E[x-K]^2 does not cancel);
//   2. finalize: one thread per channel folds the slices in float64, derives mean / 1/std and the
//      small per-channel outputs, and writes a per-channel coefficient table;
//   3. apply: a flat 128-bit streaming pass over the tensor using the table.
#include "common.h"
#include "pool2x2.h"

namespace {

using namespace dopt;

constexpr int kBlock = 256;
constexpr int kUnroll = 4;
constexpr int kMaxSlices = 64;

struct Coef {  // one per channel, 16 bytes
    float mean;  // batch (or running) mean
    float a;     // scale * rstd
    float b;     // bias
    float mean_lo;  // mean - (float)mean: keeps x - mean accurate when |mean| >> std
};
struct CoefG {   // grad: a = scale * rstd, b = dbias / m, d = dscale / m
    float mean, rstd, a, b, d, mean_lo;
    float pad[2];
};

__device__ inline float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// Fused ReLU: forward clamps the normalised value; backward drops the gradient where the ReLU
// output y is not positive (the same tests as the stand-alone relu / reluGrad kernels).
__device__ inline float relu1(float v) { return v < 0.0f ? 0.0f : v; }
__device__ inline float masked(float g, float y) { return y > 0.0f ? g : 0.0f; }
__device__ inline float4 masked4(float4 g, float4 y)
{
    return make_float4(masked(g.x, y.x), masked(g.y, y.y), masked(g.z, y.z), masked(g.w, y.w));
}

// A 2 x 2 max-pool riding on the quads of a register-resident batch norm: forward, the pooled value of the
// kernel's own output y is written as well; backward, dy is not read but made from the gradient of the
// pooled tensor, routed to the element of y the pool selected.  A lane holds four consecutive values of
// one image row; the other row of its two windows sits `wq` lanes away in the same wavefront (wq = W / 4
// quads per row, a power of two below 64; the kernels' quad index has the lane in its low six bits and
// planes are whole pairs of rows), so one exchange per quad serves both rows.  mode 2: the images are
// 2 x 2, a quad is a whole image and its own window.
struct Pool {
    int mode;             // 0: no pooling; 1: rows of quads; 2: 2 x 2 images
    unsigned wq, wshift;  // quads per image row and its log2 (mode 1)
    float *pooled;        // forward: [N, C, H/2, W/2]
    const float *dpool;   // backward: gradient of that tensor
    // backward, dsplits > 1: the gradient still lies in `dsplits` partial copies, `dstride` floats apart, the first
    // at dpool; the kernel adds them in order as it routes them and writes the sum to dvalue unless that is null
    unsigned dsplits;
    size_t dstride;
    float *dvalue;
};

// The value at `at` (in units of V) of a pooled gradient that may still lie in partial copies: copy 0 + copy 1 + ...
// in that order, up to four loads in flight (indices clamped to the last copy, surplus values dropped).
template <typename V>
__device__ inline V pool_dvalue(const Pool &pl, size_t at, bool write)
{
    const V *src = (const V *)pl.dpool + at;
    if (pl.dsplits <= 1) return *src;
    const size_t stride = pl.dstride / (sizeof(V) / sizeof(float));
    const unsigned last = pl.dsplits - 1;
    V acc = src[0];
    for (unsigned s = 1; s <= last; s += 4) {
        const unsigned s1 = min(s + 1, last), s2 = min(s + 2, last), s3 = min(s + 3, last);
        const V v0 = src[(size_t)s * stride], v1 = src[(size_t)s1 * stride], v2 = src[(size_t)s2 * stride], v3 = src[(size_t)s3 * stride];
        if constexpr (sizeof(V) == sizeof(float)) {
            acc += v0;
            if (s + 1 <= last) acc += v1;
            if (s + 2 <= last) acc += v2;
            if (s + 3 <= last) acc += v3;
        } else {
            acc.x += v0.x; acc.y += v0.y;
            if (s + 1 <= last) { acc.x += v1.x; acc.y += v1.y; }
            if (s + 2 <= last) { acc.x += v2.x; acc.y += v2.y; }
            if (s + 3 <= last) { acc.x += v3.x; acc.y += v3.y; }
        }
    }
    if (write && pl.dvalue) ((V *)pl.dvalue)[at] = acc;
    return acc;
}

__device__ inline float4 quad_xor(float4 v, unsigned lanes)
{
    return make_float4(__shfl_xor(v.x, (int)lanes, 64), __shfl_xor(v.y, (int)lanes, 64), __shfl_xor(v.z, (int)lanes, 64),
                       __shfl_xor(v.w, (int)lanes, 64));
}

// Forward: y is this lane's finished quad at float4 index idx of [N, C, H, W] (absent: idx == ~0u, y
// arbitrary).  Every lane of the wavefront must call it.  With idx = map * H * wq + h * wq + cq, idx >> wshift
// is the row index map * H + h over the whole tensor, and H is even: its parity is the row's, its half the
// pooled row.
__device__ inline void pool_store(const Pool &pl, float4 y, unsigned idx)
{
    const bool present = idx != 0xffffffffu;
    if (pl.mode == 2) {
        if (present) pl.pooled[idx] = pool2x2(y.x, y.y, y.z, y.w);
        return;
    }
    const float4 o = quad_xor(y, pl.wq);
    const unsigned row = idx >> pl.wshift, cq = idx & (pl.wq - 1);
    if (present && !(row & 1))
        ((float2 *)pl.pooled)[(size_t)(row >> 1) * pl.wq + cq] = make_float2(pool2x2(y.x, y.y, o.x, o.y), pool2x2(y.z, y.w, o.z, o.w));
}

// Backward: the quad of dy = maxpoolGrad(dpool, y) at float4 index idx, from this lane's quad of y (zeros
// when absent).  Every lane of the wavefront must call it.
__device__ inline float4 pool_grad(const Pool &pl, float4 y, unsigned idx)
{
    const bool present = idx != 0xffffffffu;
    float4 r;
    // an absent lane loads element 0 and drops it: a load under a lane mask would end in a wait of its own, and the
    // loads of a thread's quads would go out one after the other instead of together
    if (pl.mode == 2) {
        const float gl = pool_dvalue<float>(pl, present ? idx : 0u, present);
        const float g = present ? gl : 0.0f;
        route2x2(y.x, y.y, y.z, y.w, g, r.x, r.y, r.z, r.w);
        return r;
    }
    const float4 o = quad_xor(y, pl.wq);
    const unsigned row = present ? idx >> pl.wshift : 0u, cq = present ? idx & (pl.wq - 1) : 0u;
    const bool odd = row & 1;
    // both rows of a window read its gradient; the even row writes the finished sum of an open one
    const float2 gl = pool_dvalue<float2>(pl, (size_t)(row >> 1) * pl.wq + cq, present && !odd);
    const float2 g = present ? gl : make_float2(0.0f, 0.0f);
    const float4 top = odd ? o : y, bot = odd ? y : o;
    float4 t, b;
    route2x2(top.x, top.y, bot.x, bot.y, g.x, t.x, t.y, b.x, b.y);
    route2x2(top.z, top.w, bot.z, bot.w, g.y, t.z, t.w, b.z, b.w);
    return odd ? b : t;
}

// Sums four per-thread values over the block; results valid in thread 0.
__device__ inline void block_sum(float (&v)[4], float (*part)[kBlock / 64])
{
    constexpr int kN = 4;
#pragma unroll
    for (int k = 0; k < kN; k++) {
        v[k] = wave_sum(v[k]);
        if ((threadIdx.x & 63) == 0) part[k][threadIdx.x >> 6] = v[k];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int k = 0; k < kN; k++) {
            float r = 0.0f;
#pragma unroll
            for (int w = 0; w < kBlock / 64; w++) r += part[k][w];
            v[k] = r;
        }
    }
}

// Moments of x (and of dy, dy*(x-K) when kGrad) for block (c, s): images n = s, s+S, ...
// kFlat: for small `inner` the block walks (n, i) pairs with a flat index instead of rows.
template <bool kGrad, bool kFlat>
__global__ __launch_bounds__(kBlock) void bn_partial_k(size_t N, size_t C, size_t inner, size_t S, const float *x,
                                                        const float *dy, const float *ymask, float *partial)
{
    __shared__ float part[4][kBlock / 64];
    const size_t c = blockIdx.x % C, s = blockIdx.x / C;
    const float K = x[c * inner];
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (kFlat) {
        const size_t per = N * inner;
        for (size_t j = threadIdx.x; j < per; j += kBlock) {
            size_t n = j / inner, i = j % inner;
            size_t e = (n * C + c) * inner + i;
            float v = x[e] - K;
            acc[0] += v;
            acc[1] += v * v;
            if (kGrad) {
                float g = dy[e];
                if (ymask) g = masked(g, ymask[e]);
                acc[2] += g;
                acc[3] += g * v;
            }
        }
    } else {
        // inner % 4 == 0 and 16-byte aligned rows (checked on the host)
        const size_t inner4 = inner >> 2;
        for (size_t n = s; n < N; n += S) {
            const float4 *row = (const float4 *)(x + (n * C + c) * inner);
            const float4 *grow = (const float4 *)(dy + (n * C + c) * inner);
            const float4 *mrow = (const float4 *)(ymask + (n * C + c) * inner);
            for (size_t i = threadIdx.x; i < inner4; i += kBlock) {
                float4 q = row[i];
                float v0 = q.x - K, v1 = q.y - K, v2 = q.z - K, v3 = q.w - K;
                acc[0] += (v0 + v1) + (v2 + v3);
                acc[1] += (v0 * v0 + v1 * v1) + (v2 * v2 + v3 * v3);
                if (kGrad) {
                    float4 g = grow[i];
                    if (ymask) g = masked4(g, mrow[i]);
                    acc[2] += (g.x + g.y) + (g.z + g.w);
                    acc[3] += (g.x * v0 + g.y * v1) + (g.z * v2 + g.w * v3);
                }
            }
        }
    }
    block_sum(acc, part);
    if (threadIdx.x == 0) {
        float *p = partial + (c * S + s) * 4;
        p[0] = acc[0];
        p[1] = acc[1];
        if (kGrad) {
            p[2] = acc[2];
            p[3] = acc[3];
        }
    }
}

__global__ __launch_bounds__(kBlock) void bn_train_finalize_k(size_t N, size_t C, size_t inner, size_t S,
                                                               double factor, double eps, const float *x,
                                                               const float *partial, const float *scale,
                                                               const float *bias, const float *run_mean,
                                                               const float *run_var, Coef *coef, float *new_mean,
                                                               float *new_var)
{
    size_t c = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (c >= C) return;
    double m = (double)N * (double)inner;
    double s1 = 0.0, s2 = 0.0;
    for (size_t s = 0; s < S; s++) {
        s1 += (double)partial[(c * S + s) * 4 + 0];
        s2 += (double)partial[(c * S + s) * 4 + 1];
    }
    double K = (double)x[c * inner];
    double d1 = s1 / m;
    double mean = K + d1;
    double var = s2 / m - d1 * d1;  // biased
    if (var < 0.0) var = 0.0;
    double rstd = 1.0 / sqrt(var + eps);
    Coef k;
    k.mean = (float)mean;
    k.a = (float)((double)scale[c] * rstd);
    k.b = bias[c];
    k.mean_lo = (float)(mean - (double)k.mean);
    coef[c] = k;
    double unbiased = m > 1.0 ? var * m / (m - 1.0) : var;
    new_mean[c] = (float)((1.0 - factor) * (double)run_mean[c] + factor * mean);
    new_var[c] = (float)((1.0 - factor) * (double)run_var[c] + factor * unbiased);
}

__global__ __launch_bounds__(kBlock) void bn_infer_prepare_k(size_t C, double eps, const float *scale,
                                                              const float *bias, const float *mean, const float *var,
                                                              Coef *coef)
{
    size_t c = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (c >= C) return;
    double rstd = 1.0 / sqrt((double)var[c] + eps);
    Coef k;
    k.mean = mean[c];
    k.a = (float)((double)scale[c] * rstd);
    k.b = bias[c];
    k.mean_lo = 0.0f;
    coef[c] = k;
}

// Inference in one launch: block (c, slice) derives its channel's coefficients itself (one float64
// reciprocal square root per thread) and streams that channel's rows of images slice, slice + S, ...
// with four 128-bit loads in flight per thread.  Same arithmetic as the coefficient table + bn_apply_k.
__global__ __launch_bounds__(kBlock) void bn_infer_chan_k(unsigned N, unsigned C, unsigned inner4, unsigned S, double eps,
                                                           const float *x, const float *scale, const float *bias,
                                                           const float *mean, const float *var, float *y)
{
    const unsigned c = blockIdx.x % C, s = blockIdx.x / C;
    const double rstd = 1.0 / sqrt((double)var[c] + eps);
    const float m = mean[c], a = (float)((double)scale[c] * rstd), b = bias[c];
    const unsigned nimg = (N - s + S - 1) / S, tot = nimg * inner4;
    const float4 *x4 = (const float4 *)x;
    float4 *y4 = (float4 *)y;
    for (unsigned base = threadIdx.x; base < tot; base += kUnroll * kBlock) {
        float4 v[kUnroll];
        size_t at[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const unsigned t = base + u * kBlock;
            const unsigned j = t / inner4, i = t - j * inner4;
            at[u] = ((size_t)(s + j * S) * C + c) * inner4 + i;
            if (t < tot) v[u] = x4[at[u]];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            if (base + u * kBlock >= tot) continue;
            float4 r;
            r.x = a * ((v[u].x - m) - 0.0f) + b;
            r.y = a * ((v[u].y - m) - 0.0f) + b;
            r.z = a * ((v[u].z - m) - 0.0f) + b;
            r.w = a * ((v[u].w - m) - 0.0f) + b;
            y4[at[u]] = r;
        }
    }
}

__global__ __launch_bounds__(kBlock) void bn_grad_finalize_k(size_t N, size_t C, size_t inner, size_t S, double eps,
                                                              const float *x, const float *partial,
                                                              const float *scale, CoefG *coef, float *dscale,
                                                              float *dbias)
{
    size_t c = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (c >= C) return;
    double m = (double)N * (double)inner;
    double s1 = 0.0, s2 = 0.0, g1 = 0.0, g2 = 0.0;
    for (size_t s = 0; s < S; s++) {
        const float *p = partial + (c * S + s) * 4;
        s1 += (double)p[0];
        s2 += (double)p[1];
        g1 += (double)p[2];
        g2 += (double)p[3];
    }
    double K = (double)x[c * inner];
    double d1 = s1 / m;
    double mean = K + d1;
    double var = s2 / m - d1 * d1;
    if (var < 0.0) var = 0.0;
    double rstd = 1.0 / sqrt(var + eps);
    double db = g1;                          // sum dy
    double ds = rstd * (g2 - d1 * g1);       // sum dy * xhat,  xhat = (x - mean) * rstd
    CoefG k;
    k.mean = (float)mean;
    k.rstd = (float)rstd;
    k.a = (float)((double)scale[c] * rstd);
    k.b = (float)(db / m);
    k.d = (float)(ds / m);
    k.mean_lo = (float)(mean - (double)k.mean);
    k.pad[0] = k.pad[1] = 0.0f;
    coef[c] = k;
    dscale[c] = (float)ds;
    dbias[c] = (float)db;
}

// y = a * ((x - mean) - mean_lo) + b
template <typename IdxT, bool kVec>
__global__ __launch_bounds__(kBlock) void bn_apply_k(IdxT total, IdxT C, IdxT inner, const float *x, const Coef *coef,
                                                      float *y, int relu)
{
    if (kVec) {
        const IdxT n4 = total >> 2, inner4 = inner >> 2;
        const float4 *x4 = (const float4 *)x;
        float4 *y4 = (float4 *)y;
        for (IdxT base = (IdxT)blockIdx.x * (kBlock * kUnroll); base < n4;
             base += (IdxT)gridDim.x * (kBlock * kUnroll)) {
            float4 v[kUnroll];
            Coef k[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                IdxT i = base + (IdxT)u * kBlock + threadIdx.x;
                if (i < n4) {
                    v[u] = x4[i];
                    k[u] = coef[(i / inner4) % C];
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                IdxT i = base + (IdxT)u * kBlock + threadIdx.x;
                if (i < n4) {
                    float4 r;
                    r.x = k[u].a * ((v[u].x - k[u].mean) - k[u].mean_lo) + k[u].b;
                    r.y = k[u].a * ((v[u].y - k[u].mean) - k[u].mean_lo) + k[u].b;
                    r.z = k[u].a * ((v[u].z - k[u].mean) - k[u].mean_lo) + k[u].b;
                    r.w = k[u].a * ((v[u].w - k[u].mean) - k[u].mean_lo) + k[u].b;
                    if (relu) r = make_float4(relu1(r.x), relu1(r.y), relu1(r.z), relu1(r.w));
                    y4[i] = r;
                }
            }
        }
    } else {
        for (IdxT i = (IdxT)blockIdx.x * kBlock + threadIdx.x; i < total; i += (IdxT)gridDim.x * kBlock) {
            Coef k = coef[(i / inner) % C];
            const float r = k.a * ((x[i] - k.mean) - k.mean_lo) + k.b;
            y[i] = relu ? relu1(r) : r;
        }
    }
}

// dx = a * (dy - b - xhat * d),  xhat = (x - mean) * rstd
__device__ inline float bn_dx(const CoefG &k, float dy, float x)
{
    float xhat = ((x - k.mean) - k.mean_lo) * k.rstd;
    return k.a * ((dy - k.b) - xhat * k.d);
}

template <typename IdxT, bool kVec>
__global__ __launch_bounds__(kBlock) void bn_grad_apply_k(IdxT total, IdxT C, IdxT inner, const float *dy,
                                                           const float *ymask, const float *x, const CoefG *coef,
                                                           float *dx)
{
    if (kVec) {
        const IdxT n4 = total >> 2, inner4 = inner >> 2;
        const float4 *x4 = (const float4 *)x;
        const float4 *g4 = (const float4 *)dy;
        float4 *o4 = (float4 *)dx;
        for (IdxT base = (IdxT)blockIdx.x * (kBlock * kUnroll); base < n4;
             base += (IdxT)gridDim.x * (kBlock * kUnroll)) {
            float4 v[kUnroll], g[kUnroll];
            IdxT ch[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                IdxT i = base + (IdxT)u * kBlock + threadIdx.x;
                if (i < n4) {
                    v[u] = x4[i];
                    g[u] = g4[i];
                    if (ymask) g[u] = masked4(g[u], ((const float4 *)ymask)[i]);
                    ch[u] = (i / inner4) % C;
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                IdxT i = base + (IdxT)u * kBlock + threadIdx.x;
                if (i < n4) {
                    CoefG k = coef[ch[u]];
                    o4[i] = make_float4(bn_dx(k, g[u].x, v[u].x), bn_dx(k, g[u].y, v[u].y), bn_dx(k, g[u].z, v[u].z),
                                        bn_dx(k, g[u].w, v[u].w));
                }
            }
        }
    } else {
        for (IdxT i = (IdxT)blockIdx.x * kBlock + threadIdx.x; i < total; i += (IdxT)gridDim.x * kBlock) {
            CoefG k = coef[(i / inner) % C];
            dx[i] = bn_dx(k, ymask ? masked(dy[i], ymask[i]) : dy[i], x[i]);
        }
    }
}

// ---- channel-resident path -------------------------------------------------------------------
// One block per channel for tensors whose channel (N * inner values) fits the block's registers:
// x (and dy) are read ONCE, held in registers between the statistics and the output pass, and
// the op is one launch instead of three.  Statistics are exact two-pass (mean, then centred
// squares).
constexpr int kResQuads = 8;  // float4 per thread
constexpr int kOpenQuads = 2; // the same where an operand arrives as partial copies

// Sums kN per-thread values over the block (up to 16 wavefronts); every thread gets the totals.
// Lanes are folded in fp32 with butterfly shuffles (a pairwise tree: error ~ log2(64) ulp), the
// wavefront sums are added in float64 in wavefront order.  A one-wavefront block needs no LDS
// and no barrier, which is what the many small channels of the deep layers run.
template <int kN>
__device__ inline void block_allsum(const float (&v)[kN], double (&total)[kN], float (*part)[16])
{
    float w[kN];
#pragma unroll
    for (int k = 0; k < kN; k++) {
        w[k] = v[k];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) w[k] += __shfl_xor(w[k], off, 64);
    }
    const int nw = (blockDim.x + 63) >> 6;
    if (nw == 1) {
#pragma unroll
        for (int k = 0; k < kN; k++) total[k] = (double)w[k];
        return;
    }
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // `part` may still be read from the previous call
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int k = 0; k < kN; k++) part[k][wave] = w[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kN; k++) {
        double r = 0.0;
        for (int i = 0; i < nw; i++) r += (double)part[k][i];
        total[k] = r;
    }
}

// An operand that a convolution left as `splits` partial copies (x of the forward kernel, dy of the
// gradient kernel): the kernel adds the copies in order, plus the convolution's bias, exactly as the
// convolution's own finishing pass would, and writes the finished value to `value` when that is
// not null (the forward input is read again by the backward pass).
struct OpenSum {
    const float4 *partial;
    int splits;
    unsigned stride4;   // float4 per copy
    const float *bias;  // per channel, or null
    float4 *value;      // or null
};

// sum[i] = copy 0 + copy 1 + ... at float4 index at[i], in that order.  kS > 0: exactly kS copies,
// unrolled; kS == 0: any number, copy by copy with the quads of one copy in flight together.
template <int kS, int kQ>
__device__ __forceinline__ void open_add(const OpenSum &open, const unsigned (&at)[kQ], float4 (&sum)[kQ])
{
    if constexpr (kS > 0) {
        float4 v[kS][kQ];
#pragma unroll
        for (int sp = 0; sp < kS; sp++)
#pragma unroll
            for (int i = 0; i < kQ; i++) v[sp][i] = open.partial[(size_t)sp * open.stride4 + at[i]];
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            sum[i] = v[0][i];
#pragma unroll
            for (int sp = 1; sp < kS; sp++)
                sum[i] = make_float4(sum[i].x + v[sp][i].x, sum[i].y + v[sp][i].y, sum[i].z + v[sp][i].z, sum[i].w + v[sp][i].w);
        }
    } else {
        // rounds of eight copies in flight (indices clamped to the last copy, surplus values dropped); the adds stay
        // in ascending copy order
        const int last = open.splits - 1;
        for (int sp = 0; sp <= last; sp += 8) {
            float4 v[8][kQ];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const float4 *src = open.partial + (size_t)min(sp + u, last) * open.stride4;
#pragma unroll
                for (int i = 0; i < kQ; i++) v[u][i] = src[at[i]];
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (sp + u > last) break;
#pragma unroll
                for (int i = 0; i < kQ; i++) {
                    if (sp + u == 0) sum[i] = v[u][i];
                    else sum[i] = make_float4(sum[i].x + v[u][i].x, sum[i].y + v[u][i].y, sum[i].z + v[u][i].z, sum[i].w + v[u][i].w);
                }
            }
        }
    }
}

// A sum that rides along in a batch-norm launch: `splits` partial copies of n4 quads (stride n4), added by the
// workgroups from `first` on in the order of the filter gradient's own finishing pass (split_sum_k in conv.hip:
// `lanes` interleaved lanes, lane l folding copies l, l + lanes, ... in four chains that start from zero, lane
// value (a0 + a1) + (a2 + a3), lanes added in lane order, a lane without copies contributing +0).  One thread
// per quad walks the lanes one after the other with a lane's four chains in flight.
struct SideSum {
    const float4 *partial;
    float4 *out;
    unsigned n4, splits, lanes;
    unsigned first;   // 0: nothing rides
};

__device__ inline void add4(float4 &a, const float4 v)
{
    a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
}

__device__ inline void side_sum(const SideSum &sd)
{
    const unsigned L = sd.lanes, S = sd.splits;
    const size_t step = (size_t)(gridDim.x - sd.first) * blockDim.x;
    for (size_t i = (size_t)(blockIdx.x - sd.first) * blockDim.x + threadIdx.x; i < sd.n4; i += step) {
        const float4 *q = sd.partial + i;
        float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
        for (unsigned sl = 0; sl < L; sl++) {
            float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0, a2 = a0, a3 = a0;
            unsigned sp = sl;
            for (; sp + 3 * L < S; sp += 4 * L) {
                const float4 v0 = q[(size_t)sp * sd.n4], v1 = q[(size_t)(sp + L) * sd.n4];
                const float4 v2 = q[(size_t)(sp + 2 * L) * sd.n4], v3 = q[(size_t)(sp + 3 * L) * sd.n4];
                add4(a0, v0); add4(a1, v1); add4(a2, v2); add4(a3, v3);
            }
            for (; sp < S; sp += L) add4(a0, q[(size_t)sp * sd.n4]);
            const float4 lane = make_float4((a0.x + a1.x) + (a2.x + a3.x), (a0.y + a1.y) + (a2.y + a3.y),
                                            (a0.z + a1.z) + (a2.z + a3.z), (a0.w + a1.w) + (a2.w + a3.w));
            if (sl == 0) r = lane;
            else add4(r, lane);
        }
        sd.out[i] = r;
    }
}

// kQ: float4 per thread (a thread of the open variant holds kQ quads of every copy at once, so it is
// built for small channels only).
template <bool kGrad, bool kOpen, int kQ>
__global__ __launch_bounds__(1024) void bn_resident_k(unsigned N, unsigned C, unsigned inner4, double factor, double eps,
                                                       const float *x, const float *dy, const float *scale,
                                                       const float *bias, const float *run_mean, const float *run_var,
                                                       const float *ymask, int relu, float *out, float *out1, float *out2,
                                                       float *dx_sum, OpenSum open, Pool pool, SideSum side)
{
    __shared__ float part[3][16];
    if (side.first && blockIdx.x >= side.first) {   // a workgroup behind the channels': the sum that rides along
        side_sum(side);
        return;
    }
    const unsigned c = blockIdx.x, T = blockDim.x, E4 = N * inner4;
    const float4 *x4 = (const float4 *)x, *g4 = (const float4 *)dy;
    float4 xv[kQ], gv[kQ];
    unsigned idx[kQ], at[kQ];
#pragma unroll
    for (int i = 0; i < kQ; i++) {
        const unsigned q = i * T + threadIdx.x;
        const unsigned n = q / inner4, r = q - n * inner4;
        idx[i] = q < E4 ? (n * C + c) * inner4 + r : 0xffffffffu;
        at[i] = q < E4 ? idx[i] : c * inner4;   // an absent quad loads the channel's first one and drops it
    }
    // Loads are clamped, never branched, and grouped per operand: a load under a lane mask ends in a wait of its own,
    // and a thread's quads would be fetched one after the other instead of all at once.
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kQ; i++) {
        xv[i] = (kOpen && !kGrad) ? zero4 : x4[at[i]];
        gv[i] = zero4;
    }
    if (kGrad && !kOpen) {
        if (pool.mode) {
#pragma unroll
            for (int i = 0; i < kQ; i++) gv[i] = ((const float4 *)ymask)[at[i]];   // y for now; dy below
        } else {
#pragma unroll
            for (int i = 0; i < kQ; i++) gv[i] = g4[at[i]];
            if (ymask) {
                float4 mv[kQ];
#pragma unroll
                for (int i = 0; i < kQ; i++) mv[i] = ((const float4 *)ymask)[at[i]];
#pragma unroll
                for (int i = 0; i < kQ; i++) gv[i] = masked4(gv[i], mv[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kQ; i++)
        if (idx[i] == 0xffffffffu) xv[i] = gv[i] = zero4;
    if (kGrad && !kOpen && pool.mode) {   // dy = reluGrad(maxpoolGrad(dpool, y), y)
#pragma unroll
        for (int i = 0; i < kQ; i++) gv[i] = masked4(pool_grad(pool, gv[i], idx[i]), gv[i]);
    }
    if (kOpen) {
        float4 sum[kQ];
        // two to four copies: every load of the thread is issued before the first add
        if (open.splits == 2) open_add<2, kQ>(open, at, sum);
        else if (open.splits == 3) open_add<3, kQ>(open, at, sum);
        else if (open.splits == 4) open_add<4, kQ>(open, at, sum);
        else open_add<0, kQ>(open, at, sum);
        const bool biased = open.bias != nullptr;
        const float bc = biased ? open.bias[c] : 0.0f;
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            float4 r = sum[i];
            if (biased) r = make_float4(r.x + bc, r.y + bc, r.z + bc, r.w + bc);
            if (open.value) open.value[idx[i]] = r;
            if (kGrad) gv[i] = ymask ? masked4(r, ((const float4 *)ymask)[idx[i]]) : r;
            else xv[i] = r;
        }
    }
    const double m = 4.0 * (double)E4;
    double red1[1];
    {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) s += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);  // absent quads are zero
        const float in1[1] = {s};
        block_allsum<1>(in1, red1, part);
    }
    const double mean = red1[0] / m;
    const float mean_hi = (float)mean, mean_lo = (float)(mean - (double)mean_hi);
    double red3[3];
    {
        float ss = 0.f, g1 = 0.f, g2 = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            const float d0 = (xv[i].x - mean_hi) - mean_lo, d1 = (xv[i].y - mean_hi) - mean_lo;
            const float d2 = (xv[i].z - mean_hi) - mean_lo, d3 = (xv[i].w - mean_hi) - mean_lo;
            ss += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
            if (kGrad) {
                g1 += (gv[i].x + gv[i].y) + (gv[i].z + gv[i].w);
                g2 += (gv[i].x * d0 + gv[i].y * d1) + (gv[i].z * d2 + gv[i].w * d3);
            }
        }
        const float in3[3] = {ss, g1, g2};
        block_allsum<3>(in3, red3, part);
    }
    const double var = red3[0] / m;  // biased
    const double rstd = 1.0 / sqrt(var + eps);
    float4 *o4 = (float4 *)out;
    if (!kGrad) {
        const float a = (float)((double)scale[c] * rstd), b = bias[c];
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            float4 r;
            r.x = a * ((xv[i].x - mean_hi) - mean_lo) + b;
            r.y = a * ((xv[i].y - mean_hi) - mean_lo) + b;
            r.z = a * ((xv[i].z - mean_hi) - mean_lo) + b;
            r.w = a * ((xv[i].w - mean_hi) - mean_lo) + b;
            if (relu) r = make_float4(relu1(r.x), relu1(r.y), relu1(r.z), relu1(r.w));
            o4[idx[i]] = r;
            xv[i] = r;
        }
        if (pool.mode) {
#pragma unroll
            for (int i = 0; i < kQ; i++) pool_store(pool, xv[i], idx[i]);
        }
        if (threadIdx.x == 0) {
            const double unbiased = m > 1.0 ? var * m / (m - 1.0) : var;
            out1[c] = (float)((1.0 - factor) * (double)run_mean[c] + factor * mean);
            out2[c] = (float)((1.0 - factor) * (double)run_var[c] + factor * unbiased);
        }
    } else {
        const double db = red3[1], ds = rstd * red3[2];  // sum dy, sum dy * xhat
        CoefG k;
        k.mean = mean_hi;
        k.mean_lo = mean_lo;
        k.rstd = (float)rstd;
        k.a = (float)((double)scale[c] * rstd);
        k.b = (float)(db / m);
        k.d = (float)(ds / m);
        float sdx = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            const float4 r = make_float4(bn_dx(k, gv[i].x, xv[i].x), bn_dx(k, gv[i].y, xv[i].y),
                                         bn_dx(k, gv[i].z, xv[i].z), bn_dx(k, gv[i].w, xv[i].w));
            o4[idx[i]] = r;
            sdx += (r.x + r.y) + (r.z + r.w);
        }
        if (threadIdx.x == 0) {
            out1[c] = (float)ds;
            out2[c] = (float)db;
        }
        if (dx_sum) {  // the per-channel sum of dx: the bias gradient of an addBias feeding this batch norm
            const float in1[1] = {sdx};
            double red[1];
            block_allsum<1>(in1, red, part);
            if (threadIdx.x == 0) dx_sum[c] = (float)red[0];
        }
    }
}

// ---- cluster-resident path -------------------------------------------------------------------
// Channels too large for one block's registers but small enough for a few blocks' (up to kMaxCluster x
// 32768 values: the first VGG layers at batch 128 hold 131072 values per channel): S consecutive
// blocks share a channel, each keeps its piece in registers, and the pieces' statistics meet once in
// device memory.  x (and dy) are still read once and the op is still one launch.
//
// Every block publishes (the mean it centred on, centred squares about that mean, sum dy,
// sum dy*(x - that mean)) and waits for its S - 1 partners; all of them then fold the S records in
// block order in float64 (M2 = sum of M2_j + n_j (mean_j - mean)^2, the pairwise update of Chan et
// al.), so every block of a channel derives bit-identical statistics and the result does not depend
// on arrival order.
//
// What travels between blocks are single 64-bit words written and read with device-scope atomics: a
// double as its (high float, low float) pair, 48 significant bits, with all-ones standing for "not
// there yet".  Value and presence arrive together, so no fence is needed (a release fence would first
// push everything the compute unit's cache holds out to memory).  The last block to leave a channel
// puts its words back to all-ones, so a launch -- or a replay of a recorded launch -- always starts
// from "nothing there".
//
// The wait is safe because partners have consecutive block ids (workgroups are dispatched in id order,
// so a waiting block only ever waits for blocks that are already resident or next in line, and a
// cluster needs at most kMaxCluster of the machine's CUs), and it is bounded: a block that gives up
// raises `error`, finishes with whatever it found and exits; the host reports the error at the next
// synchronisation point and re-initialises the words.
constexpr unsigned kMaxCluster = 16;
constexpr unsigned kClusterRecs = 16384;      // records (channel x piece) one launch may use
constexpr unsigned kClusterChannels = 16384;
constexpr unsigned long long kAbsent = ~0ull;

struct ClusterMem {
    unsigned long long *rec;   // [C * S][4]: centre, m2, g1, g2 of a piece
    unsigned long long *sdx;   // [C * S]: per-piece sums of dx, each one word {1, float bits}; 0 = not there yet
    unsigned *depart;          // [C]
    int *error;
};
static __device__ __align__(256) unsigned long long g_cl_rec[kClusterRecs * 4];
static __device__ __align__(256) unsigned long long g_cl_sdx[kClusterRecs];
static __device__ __align__(256) unsigned g_cl_depart[kClusterChannels];
static __device__ int g_cl_error;

__device__ inline unsigned long long pack_double(double d)
{
    float hi = (float)d;
    float lo = (float)(d - (double)hi);
    unsigned h = __float_as_uint(hi), l = __float_as_uint(lo);
    if (hi != hi) { h = 0x7fc00000u; l = 0u; }     // any NaN travels as the canonical one: never as "absent"
    return ((unsigned long long)h << 32) | l;
}
__device__ inline double unpack_double(unsigned long long w)
{
    return (double)__uint_as_float((unsigned)(w >> 32)) + (double)__uint_as_float((unsigned)w);
}

template <bool kGrad>
__global__ __launch_bounds__(1024) void bn_cluster_k(unsigned N, unsigned C, unsigned inner4, unsigned S, unsigned per,
                                                      double factor, double eps, const float *x, const float *dy,
                                                      const float *scale, const float *bias, const float *run_mean,
                                                      const float *run_var, const float *ymask, int relu, float *out,
                                                      float *out1, float *out2, float *dx_sum, ClusterMem cm,
                                                      unsigned spin_limit, Pool pool, SideSum side)
{
    constexpr int kQ = kResQuads;
    __shared__ float part[3][16];
    __shared__ double comb[4];
    if (side.first && blockIdx.x >= side.first) {   // behind every cluster: the sum that rides along (waits for no one)
        side_sum(side);
        return;
    }
    const unsigned c = blockIdx.x / S, piece = blockIdx.x - c * S, T = blockDim.x, E4 = N * inner4;
    const unsigned q0 = piece * per;                                  // this block's quads: [q0, q0 + mine)
    const unsigned mine = E4 - q0 < per ? E4 - q0 : per;
    const float4 *x4 = (const float4 *)x, *g4 = (const float4 *)dy;
    float4 xv[kQ], gv[kQ];
    unsigned idx[kQ], at[kQ];
#pragma unroll
    for (int i = 0; i < kQ; i++) {
        const unsigned l = i * T + threadIdx.x;
        const unsigned q = q0 + l;
        const unsigned n = q / inner4, r = q - n * inner4;
        idx[i] = l < mine ? (n * C + c) * inner4 + r : 0xffffffffu;
        at[i] = l < mine ? idx[i] : c * inner4;   // an absent quad loads the channel's first one and drops it
    }
    // clamped, never branched, grouped per operand: all of a thread's loads are in flight together (see bn_resident_k)
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kQ; i++) {
        xv[i] = x4[at[i]];
        gv[i] = zero4;
    }
    if (kGrad) {
        if (pool.mode) {
#pragma unroll
            for (int i = 0; i < kQ; i++) gv[i] = ((const float4 *)ymask)[at[i]];   // y for now; dy below
        } else {
#pragma unroll
            for (int i = 0; i < kQ; i++) gv[i] = g4[at[i]];
            if (ymask) {
                float4 mv[kQ];
#pragma unroll
                for (int i = 0; i < kQ; i++) mv[i] = ((const float4 *)ymask)[at[i]];
#pragma unroll
                for (int i = 0; i < kQ; i++) gv[i] = masked4(gv[i], mv[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kQ; i++)
        if (idx[i] == 0xffffffffu) xv[i] = gv[i] = zero4;
    if (kGrad && pool.mode) {   // dy = reluGrad(maxpoolGrad(dpool, y), y)
#pragma unroll
        for (int i = 0; i < kQ; i++) gv[i] = masked4(pool_grad(pool, gv[i], idx[i]), gv[i]);
    }
    // the piece's own statistics: exact two-pass, as in the one-block kernel
    const double nb = 4.0 * (double)mine;
    double red1[1];
    {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) sum += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
        const float in1[1] = {sum};
        block_allsum<1>(in1, red1, part);
    }
    const double mu = red1[0] / nb;
    const float mu_hi = (float)mu, mu_lo = (float)(mu - (double)mu_hi);
    double red3[3];
    {
        float ss = 0.f, g1 = 0.f, g2 = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            const float d0 = (xv[i].x - mu_hi) - mu_lo, d1 = (xv[i].y - mu_hi) - mu_lo;
            const float d2 = (xv[i].z - mu_hi) - mu_lo, d3 = (xv[i].w - mu_hi) - mu_lo;
            ss += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
            if (kGrad) {
                g1 += (gv[i].x + gv[i].y) + (gv[i].z + gv[i].w);
                g2 += (gv[i].x * d0 + gv[i].y * d1) + (gv[i].z * d2 + gv[i].w * d3);
            }
        }
        const float in3[3] = {ss, g1, g2};
        block_allsum<3>(in3, red3, part);
    }
    // publish, meet the partners, fold their records in block order.  The first word of a record is the
    // mean the piece centred on (exactly the float pair it used), then its moments about that mean.
    if (threadIdx.x < 4) {
        const double centre = (double)mu_hi + (double)mu_lo;
        const double mineVal = threadIdx.x == 0 ? centre : red3[threadIdx.x - 1];
        __hip_atomic_store(cm.rec + (size_t)(c * S + piece) * 4 + threadIdx.x, pack_double(mineVal), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    if (threadIdx.x < 64) {
        // lane l fetches word l of the channel's 4 * S (at most 64): all of them are polled side by side
        const unsigned nwords = 4 * S;
        unsigned long long w = 0;
        if (threadIdx.x < nwords) {
            w = kAbsent;
            for (unsigned spin = 0; spin <= spin_limit; spin++) {
                w = __hip_atomic_load(cm.rec + (size_t)c * S * 4 + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (w != kAbsent) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (w == kAbsent) __hip_atomic_store(cm.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        const double val = unpack_double(w);
        // every lane folds the same records in the same order
        const double m = 4.0 * (double)E4;
        double total = 0.0;
        for (unsigned j = 0; j < S; j++) {
            const unsigned qj = j * per;
            const double nj = 4.0 * (double)(E4 - qj < per ? E4 - qj : per);
            total += nj * __shfl(val, (int)(4 * j), 64);
        }
        const double mean = total / m;
        double m2 = 0.0, g1 = 0.0, g2 = 0.0;
        for (unsigned j = 0; j < S; j++) {
            const unsigned qj = j * per;
            const double nj = 4.0 * (double)(E4 - qj < per ? E4 - qj : per);
            const double dm = __shfl(val, (int)(4 * j), 64) - mean;
            const double rg1 = __shfl(val, (int)(4 * j + 2), 64);
            m2 += __shfl(val, (int)(4 * j + 1), 64) + nj * dm * dm;
            g1 += rg1;
            g2 += __shfl(val, (int)(4 * j + 3), 64) + dm * rg1;
        }
        if (threadIdx.x == 0) {
            comb[0] = mean;
            comb[1] = m2;
            comb[2] = g1;
            comb[3] = g2;
            // the last block to leave puts the channel's words back to "not there" for the next launch
            const unsigned left = __hip_atomic_fetch_add(cm.depart + c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (left == S - 1) {
                for (unsigned k = 0; k < nwords; k++)
                    __hip_atomic_store(cm.rec + (size_t)c * S * 4 + k, kAbsent, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(cm.depart + c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();
    const double m = 4.0 * (double)E4;
    const double mean = comb[0];
    const float mean_hi = (float)mean, mean_lo = (float)(mean - (double)mean_hi);
    const double var = comb[1] / m;  // biased
    const double rstd = 1.0 / sqrt(var + eps);
    float4 *o4 = (float4 *)out;
    if (!kGrad) {
        const float a = (float)((double)scale[c] * rstd), b = bias[c];
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            float4 r;
            r.x = a * ((xv[i].x - mean_hi) - mean_lo) + b;
            r.y = a * ((xv[i].y - mean_hi) - mean_lo) + b;
            r.z = a * ((xv[i].z - mean_hi) - mean_lo) + b;
            r.w = a * ((xv[i].w - mean_hi) - mean_lo) + b;
            if (relu) r = make_float4(relu1(r.x), relu1(r.y), relu1(r.z), relu1(r.w));
            o4[idx[i]] = r;
            xv[i] = r;
        }
        if (pool.mode) {
#pragma unroll
            for (int i = 0; i < kQ; i++) pool_store(pool, xv[i], idx[i]);
        }
        if (threadIdx.x == 0 && piece == 0) {
            const double unbiased = m > 1.0 ? var * m / (m - 1.0) : var;
            out1[c] = (float)((1.0 - factor) * (double)run_mean[c] + factor * mean);
            out2[c] = (float)((1.0 - factor) * (double)run_var[c] + factor * unbiased);
        }
    } else {
        const double db = comb[2], ds = rstd * comb[3];  // sum dy, sum dy * xhat
        CoefG k;
        k.mean = mean_hi;
        k.mean_lo = mean_lo;
        k.rstd = (float)rstd;
        k.a = (float)((double)scale[c] * rstd);
        k.b = (float)(db / m);
        k.d = (float)(ds / m);
        float sdx = 0.f;
#pragma unroll
        for (int i = 0; i < kQ; i++) {
            if (idx[i] == 0xffffffffu) continue;
            const float4 r = make_float4(bn_dx(k, gv[i].x, xv[i].x), bn_dx(k, gv[i].y, xv[i].y),
                                         bn_dx(k, gv[i].z, xv[i].z), bn_dx(k, gv[i].w, xv[i].w));
            o4[idx[i]] = r;
            sdx += (r.x + r.y) + (r.z + r.w);
        }
        if (threadIdx.x == 0 && piece == 0) {
            out1[c] = (float)ds;
            out2[c] = (float)db;
        }
        if (dx_sum) {
            // Per-channel sum of dx: piece 0 adds the pieces' sums in piece order.  A piece's sum travels as ONE
            // 64-bit word {1, float bits} written and read with device-scope atomics: value and "it is there"
            // arrive together, so no fence has to push the 128 KB of dx this block has just stored out of the
            // cache first.  Piece 0 puts the words back to 0 for the next launch.
            const float in1[1] = {sdx};
            double red[1];
            block_allsum<1>(in1, red, part);
            if (threadIdx.x == 0) {
                const unsigned long long word = (1ull << 32) | (unsigned long long)__float_as_uint((float)red[0]);
                __hip_atomic_store(cm.sdx + c * S + piece, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (piece == 0) {
                    double t = 0.0;
                    for (unsigned j = 0; j < S; j++) {
                        unsigned long long w = 0;
                        for (unsigned spin = 0; spin <= spin_limit; spin++) {
                            w = __hip_atomic_load(cm.sdx + c * S + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            if (w >> 32) break;
                            __builtin_amdgcn_s_sleep(4);
                        }
                        if (!(w >> 32)) __hip_atomic_store(cm.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        t += (double)__uint_as_float((unsigned)w);
                        __hip_atomic_store(cm.sdx + c * S + j, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    dx_sum[c] = (float)t;
                }
            }
        }
    }
}

// Host side of the cluster path: the device addresses of its records and counters (taken once per
// device), whether a launch is outstanding whose error flag has not been read, and the spin limit.
ClusterMem g_cluster_mem[64];
bool g_cluster_ready[64];
bool g_cluster_unchecked = false;
unsigned g_cluster_spin_limit = 1u << 21;   // polls of ~1 us each (2 s in all) before a block gives up

unsigned long g_cluster_launches = 0;

// The addresses and the one-time fill are made by dopt_hip_init (bn_device_setup below); a call only looks them up.
int cluster_mem(ClusterMem *out)
{
    int dev = -1;
    DOPT_HIP_CHECK(hipGetDevice(&dev));
    DOPT_REQUIRE(dev >= 0 && dev < 64, "batch norm: device index %d out of range", dev);
    DOPT_REQUIRE(g_cluster_ready[dev], "batch norm: device %d was not set up by dopt_hip_init", dev);
    *out = g_cluster_mem[dev];
    return DOPT_HIP_OK;
}

// Pieces per channel for the cluster path and quads per piece, or 0 when the tensor does not take it.
// (Channels that fit one block stay there even when they are too few to give every compute unit a
// block: 128 channels of 32768 values as 256 half-channel blocks measured 16.5 against 11.6 us forward, and the
// gradient kernels of the VGG step 10 us slower per step in all.)
unsigned cluster_pieces(size_t N, size_t C, size_t inner, const void *a, const void *b, const void *m, const void *o,
                        unsigned *per)
{
    if ((inner & 3) != 0 || !aligned16(a) || (b && !aligned16(b)) || (m && !aligned16(m)) || !aligned16(o)) return 0;
    const size_t E4 = N * (inner / 4), cap = (size_t)kResQuads * 1024;
    if (E4 <= cap || E4 > cap * kMaxCluster || N * C * (inner / 4) >= 0xffffffffull) return 0;
    const size_t S = ceil_div(E4, cap);
    if (C > kClusterChannels || C * S > kClusterRecs) return 0;
    *per = (unsigned)ceil_div(E4, S);          // balanced pieces
    return (unsigned)S;
}

// Threads for the resident path, or 0 when the channel does not fit (or is not 128-bit addressable).
unsigned resident_threads(size_t N, size_t C, size_t inner, const void *a, const void *b, const void *o)
{
    if ((inner & 3) != 0 || !aligned16(a) || (b && !aligned16(b)) || !aligned16(o)) return 0;
    const size_t E4 = N * (inner / 4);
    if (E4 == 0 || E4 > (size_t)kResQuads * 1024 || N * C * (inner / 4) >= 0xffffffffull) return 0;
    // two quads per thread where the channel is small enough: more wavefronts in flight per CU
    size_t T = (ceil_div(E4, (size_t)2) + 63) / 64 * 64;
    if (T > 1024) T = 1024;
    return (unsigned)(T < 64 ? 64 : T);
}

size_t pick_slices(size_t N, size_t C)
{
    size_t S = ceil_div((size_t)num_cus() * 8, C);
    if (S > N) S = N;
    if (S > kMaxSlices) S = kMaxSlices;
    return S < 1 ? 1 : S;
}

unsigned apply_grid(size_t total, bool vec)
{
    size_t blocks = vec ? ceil_div(total / 4, (size_t)kBlock * kUnroll) : ceil_div(total, (size_t)kBlock);
    size_t cap = (size_t)num_cus() * 8;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

template <bool kGrad>
int launch_partial(size_t N, size_t C, size_t inner, const float *x, const float *dy, const float *ymask,
                   float *partial, size_t *S_out)
{
    bool rows = inner >= 256 && (inner & 3) == 0 && aligned16(x) && (!kGrad || aligned16(dy)) &&
                (!ymask || aligned16(ymask));
    size_t S = rows ? pick_slices(N, C) : 1;
    *S_out = S;
    if (rows)
        hipLaunchKernelGGL((bn_partial_k<kGrad, false>), dim3((unsigned)(C * S)), dim3(kBlock), 0, stream(), N, C, inner,
                           S, x, dy, ymask, partial);
    else
        hipLaunchKernelGGL((bn_partial_k<kGrad, true>), dim3((unsigned)C), dim3(kBlock), 0, stream(), N, C, inner, S, x,
                           dy, ymask, partial);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int launch_apply(size_t total, size_t C, size_t inner, const float *x, const Coef *coef, float *y, int relu)
{
    bool vec = (inner & 3) == 0 && aligned16(x) && aligned16(y);
    unsigned grid = apply_grid(total, vec);
    bool small = total < 0x7fffffffull;
    if (small) {
        if (vec)
            hipLaunchKernelGGL((bn_apply_k<unsigned, true>), dim3(grid), dim3(kBlock), 0, stream(), (unsigned)total,
                               (unsigned)C, (unsigned)inner, x, coef, y, relu);
        else
            hipLaunchKernelGGL((bn_apply_k<unsigned, false>), dim3(grid), dim3(kBlock), 0, stream(), (unsigned)total,
                               (unsigned)C, (unsigned)inner, x, coef, y, relu);
    } else {
        if (vec)
            hipLaunchKernelGGL((bn_apply_k<size_t, true>), dim3(grid), dim3(kBlock), 0, stream(), total, C, inner, x,
                               coef, y, relu);
        else
            hipLaunchKernelGGL((bn_apply_k<size_t, false>), dim3(grid), dim3(kBlock), 0, stream(), total, C, inner, x,
                               coef, y, relu);
    }
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// The kernel-side description of an open operand, or false when `o` does not describe `elems` values
// in [N, C, inner] that the resident kernel can read (the caller then closes it first).
bool open_sum(const dopt_hip_split_sum *o, size_t elems, size_t C, size_t inner, bool keep, OpenSum *k)
{
    if (!o || o->splits < 2 || o->elems != elems || o->C != C || o->inner != inner || !o->partial || !o->value ||
        !aligned16(o->partial) || !aligned16(o->value) || elems % 4 != 0)
        return false;
    k->partial = (const float4 *)o->partial;
    k->splits = o->splits;
    k->stride4 = (unsigned)(elems / 4);
    k->bias = o->bias;
    k->value = keep ? (float4 *)o->value : nullptr;
    return true;
}

// What the caller wants pooled (null: nothing) and whether the register-resident kernels can do it on the way:
// images of W = 4 .. 128 (a power of two) by an even H, or 2 x 2 images.
struct PoolArg {
    size_t H, W;
    float *pooled;        // forward
    const float *dpool;   // backward
    const dopt_hip_split_sum *dopen = nullptr;   // backward: dpool still lies in partial copies (or null)
    bool keep = true;                            // ... and its finished value is wanted as well
};

bool pool_inline(const PoolArg *a, Pool *k)
{
    *k = Pool{};
    if (!a) return false;
    const void *ptr = a->pooled ? (const void *)a->pooled : (const void *)a->dpool;
    if (a->H == 2 && a->W == 2) {
        k->mode = 2;
    } else if (a->W >= 4 && a->W <= 128 && (a->W & (a->W - 1)) == 0 && (a->H & 1) == 0 && ((uintptr_t)ptr & 7) == 0) {
        k->mode = 1;
        k->wq = (unsigned)(a->W / 4);
        k->wshift = (unsigned)__builtin_ctz(k->wq);
    } else {
        return false;
    }
    k->pooled = a->pooled;
    k->dpool = a->dpool;
    return true;
}

int bn_train_impl(size_t N, size_t C, size_t inner, double momentum, const float *x, const float *scale,
                  const float *bias, const float *run_mean, const float *run_var, float *packed, int relu,
                  const char *who, const dopt_hip_split_sum *x_open = nullptr, const PoolArg *pool = nullptr)
{
    size_t total = N * C * inner;
    Pool pl;
    const bool pool_in = pool_inline(pool, &pl);   // a resident kernel pools on the way; else a pass of its own follows
    auto pooled_after = [&]() -> int {
        return pool ? dopt_hip_maxpool_fwd(N, C, pool->H, pool->W, 2, 2, packed, pool->pooled) : DOPT_HIP_OK;
    };
    DOPT_REQUIRE(total > 0, "%s: empty input", who);
    DOPT_REQUIRE(x && scale && bias && run_mean && run_var && packed, "%s: null argument", who);
    DOPT_REQUIRE(C <= 0x7fffffffu / kMaxSlices, "%s: too many channels", who);
    DOPT_ENSURE_INIT();
    double factor = 1.0 - momentum;    // cudnn7.d:592
    double eps = (double)1e-5f;        // cudnn7.d:610
    const unsigned T = resident_threads(N, C, inner, x, nullptr, packed);
    if (x_open && x_open->splits) {   // x is still in pieces
        OpenSum os;
        if (T && N * (inner / 4) <= (size_t)kOpenQuads * T && open_sum(x_open, total, C, inner, true, &os)) {
            open_split_clear(x_open->partial);
            hipLaunchKernelGGL((bn_resident_k<false, true, kOpenQuads>), dim3((unsigned)C), dim3(T), 0, stream(), (unsigned)N, (unsigned)C,
                               (unsigned)(inner / 4), factor, eps, x, (const float *)nullptr, scale, bias, run_mean, run_var,
                               (const float *)nullptr, relu, packed, packed + total, packed + total + C, (float *)nullptr, os,
                               pool_in ? pl : Pool{}, SideSum{});
            DOPT_LAUNCH_CHECK();
            return pool_in ? DOPT_HIP_OK : pooled_after();
        }
        if (int rc = dopt_hip_split_sum_close(x_open)) return rc;
    }
    unsigned per = 0;
    if (const unsigned S = cluster_pieces(N, C, inner, x, nullptr, nullptr, packed, &per)) {
        ClusterMem cm;
        if (int rc = cluster_mem(&cm)) return rc;
        const bool in = pool_in && (pl.mode == 2 || per % (2 * pl.wq) == 0);   // pieces hold whole pairs of rows
        hipLaunchKernelGGL((bn_cluster_k<false>), dim3((unsigned)(C * S)), dim3(1024), 0, stream(), (unsigned)N, (unsigned)C,
                           (unsigned)(inner / 4), S, per, factor, eps, x, (const float *)nullptr, scale, bias, run_mean,
                           run_var, (const float *)nullptr, relu, packed, packed + total, packed + total + C,
                           (float *)nullptr, cm, g_cluster_spin_limit, in ? pl : Pool{}, SideSum{});
        DOPT_LAUNCH_CHECK();
        g_cluster_unchecked = true;
        g_cluster_launches++;
        return in ? DOPT_HIP_OK : pooled_after();
    }
    if (T) {
        // small channels (two quads per thread) take the variant built for two: a third of the registers
        if (N * (inner / 4) <= (size_t)kOpenQuads * T)
            hipLaunchKernelGGL((bn_resident_k<false, false, kOpenQuads>), dim3((unsigned)C), dim3(T), 0, stream(), (unsigned)N,
                               (unsigned)C, (unsigned)(inner / 4), factor, eps, x, (const float *)nullptr, scale, bias, run_mean,
                               run_var, (const float *)nullptr, relu, packed, packed + total, packed + total + C,
                               (float *)nullptr, OpenSum{}, pool_in ? pl : Pool{}, SideSum{});
        else
            hipLaunchKernelGGL((bn_resident_k<false, false, kResQuads>), dim3((unsigned)C), dim3(T), 0, stream(), (unsigned)N,
                               (unsigned)C, (unsigned)(inner / 4), factor, eps, x, (const float *)nullptr, scale, bias, run_mean,
                               run_var, (const float *)nullptr, relu, packed, packed + total, packed + total + C,
                               (float *)nullptr, OpenSum{}, pool_in ? pl : Pool{}, SideSum{});
        DOPT_LAUNCH_CHECK();
        return pool_in ? DOPT_HIP_OK : pooled_after();
    }
    // workspace: [partials C*S*4 floats | coefficient table C * 16 bytes]
    size_t part_bytes = C * kMaxSlices * 4 * sizeof(float);
    char *ws = (char *)workspace(part_bytes + C * sizeof(Coef));
    if (!ws) return DOPT_HIP_ERR_OOM;
    float *partial = (float *)ws;
    Coef *coef = (Coef *)(ws + part_bytes);
    size_t S;
    if (int rc = launch_partial<false>(N, C, inner, x, nullptr, nullptr, partial, &S)) return rc;
    hipLaunchKernelGGL(bn_train_finalize_k, dim3((unsigned)ceil_div(C, (size_t)kBlock)), dim3(kBlock), 0, stream(), N,
                       C, inner, S, factor, eps, x, partial, scale, bias, run_mean, run_var, coef, packed + total,
                       packed + total + C);
    DOPT_LAUNCH_CHECK();
    if (int rc = launch_apply(total, C, inner, x, coef, packed, relu)) return rc;
    return pooled_after();
}

// The kernel-side description of a sum that rides along, for a launch whose own workgroups are `own` of `T`
// threads: false when `side` is null, complete or not of that kind (the caller closes it first).
bool side_sum_arg(const dopt_hip_split_sum *side, unsigned own, unsigned T, SideSum *k, unsigned *blocks)
{
    *k = SideSum{};
    *blocks = 0;
    if (!side || side->splits < 2 || side->lanes <= 0 || !side->partial || !side->value || side->elems % 4 != 0 ||
        !aligned16(side->partial) || !aligned16(side->value) || side->elems / 4 >= 0xffffffffull || own == 0 || T == 0)
        return false;
    k->partial = (const float4 *)side->partial;
    k->out = (float4 *)side->value;
    k->n4 = (unsigned)(side->elems / 4);
    k->splits = (unsigned)side->splits;
    k->lanes = (unsigned)side->lanes;
    k->first = own;
    // one quad per thread, at most 1024 threads' worth per compute unit (the loop strides beyond that)
    const size_t want = ceil_div((size_t)k->n4, (size_t)T), cap = ceil_div((size_t)num_cus() * 1024, (size_t)T);
    *blocks = (unsigned)(want < cap ? want : cap);
    return true;
}

int bn_grad_impl(size_t N, size_t C, size_t inner, const float *dy, const float *ymask, const float *x,
                 const float *scale, float *packed, float *dx_sum, const char *who,
                 const dopt_hip_split_sum *dy_open = nullptr, bool keep_dy = true, const PoolArg *pool = nullptr,
                 const dopt_hip_split_sum *side = nullptr)
{
    size_t total = N * C * inner;
    DOPT_REQUIRE(total > 0, "%s: empty input", who);
    DOPT_REQUIRE((dy || pool) && x && scale && packed, "%s: null argument", who);
    DOPT_REQUIRE(C <= 0x7fffffffu / kMaxSlices, "%s: too many channels", who);
    DOPT_ENSURE_INIT();
    double eps = (double)1e-5f;  // cudnn7.d:634
    unsigned T = (!ymask || aligned16(ymask)) ? resident_threads(N, C, inner, x, dy, packed) : 0;
    unsigned per = 0;
    const unsigned clusterS = cluster_pieces(N, C, inner, x, pool ? nullptr : dy, ymask, packed, &per);
    // A sum that rides along does so in the launch of a register-resident kernel; the other paths (which use the
    // workspace its copies lie in) finish it first.
    if (side && side->splits) {
        DOPT_REQUIRE(side->splits > 1 && side->lanes > 0 && side->partial && side->value, "%s: malformed side sum", who);
        SideSum probe;
        unsigned nb;
        if (!(clusterS || T) || !side_sum_arg(side, 1, 64, &probe, &nb)) {
            if (int rc = dopt_hip_split_sum_close(side)) return rc;
            side = nullptr;
        }
    } else {
        side = nullptr;
    }
    SideSum sd{};
    unsigned side_blocks = 0;
    auto with_side = [&](unsigned own, unsigned threads) {   // grid of a launch whose own workgroups are `own`
        if (side && side_sum_arg(side, own, threads, &sd, &side_blocks)) open_split_clear(side->partial);
        return dim3(own + side_blocks);
    };
    Pool pl{};
    if (pool) {
        // dy = maxpoolGrad(dpool, y): made inside a register-resident kernel where one will run, else by a pass
        // of its own into the output buffer, which every path below may read as dy while it writes dx (each
        // thread reads its elements before it writes them)
        const bool in = pool_inline(pool, &pl) && (clusterS ? (pl.mode == 2 || per % (2 * pl.wq) == 0) : T != 0);
        const dopt_hip_split_sum *dopen = pool->dopen && pool->dopen->splits ? pool->dopen : nullptr;
        if (dopen) {
            // the kernel adds the copies itself where it routes the gradient anyway; else they are added first
            const size_t pelems = total / 4;
            const bool ok = in && dopen->splits > 1 && dopen->lanes == 0 && dopen->elems == pelems && !dopen->bias &&
                            dopen->partial && dopen->value == pool->dpool && pelems % 4 == 0 && aligned16(dopen->partial) &&
                            aligned16(dopen->value);
            if (ok) {
                open_split_clear(dopen->partial);
                pl.dpool = dopen->partial;
                pl.dsplits = (unsigned)dopen->splits;
                pl.dstride = pelems;
                pl.dvalue = pool->keep ? dopen->value : nullptr;
            } else if (int rc = dopt_hip_split_sum_close(dopen)) {
                return rc;
            }
        }
        if (!in) {
            pl = Pool{};
            if (int rc = dopt_hip_maxpool_bwd(N, C, pool->H, pool->W, 2, 2, pool->dpool, ymask, packed)) return rc;
            dy = packed;
        }
    }
    if (dy_open && dy_open->splits) {   // dy is still in pieces
        OpenSum os;
        if (T && N * (inner / 4) <= (size_t)kOpenQuads * T && open_sum(dy_open, total, C, inner, keep_dy, &os)) {
            open_split_clear(dy_open->partial);
            const dim3 grid = with_side((unsigned)C, T);
            hipLaunchKernelGGL((bn_resident_k<true, true, kOpenQuads>), grid, dim3(T), 0, stream(), (unsigned)N, (unsigned)C,
                               (unsigned)(inner / 4), 0.0, eps, x, dy, scale, (const float *)nullptr,
                               (const float *)nullptr, (const float *)nullptr, ymask, 0, packed, packed + total,
                               packed + total + C, dx_sum, os, Pool{}, sd);
            DOPT_LAUNCH_CHECK();
            return DOPT_HIP_OK;
        }
        if (int rc = dopt_hip_split_sum_close(dy_open)) return rc;
    }
    if (const unsigned S = cluster_pieces(N, C, inner, x, dy, ymask, packed, &per)) {
        ClusterMem cm;
        if (int rc = cluster_mem(&cm)) return rc;
        const dim3 grid = with_side((unsigned)(C * S), 1024);
        hipLaunchKernelGGL((bn_cluster_k<true>), grid, dim3(1024), 0, stream(), (unsigned)N, (unsigned)C,
                           (unsigned)(inner / 4), S, per, 0.0, eps, x, dy, scale, (const float *)nullptr,
                           (const float *)nullptr, (const float *)nullptr, ymask, 0, packed, packed + total,
                           packed + total + C, dx_sum, cm, g_cluster_spin_limit, pl, sd);
        DOPT_LAUNCH_CHECK();
        g_cluster_unchecked = true;
        g_cluster_launches++;
        return DOPT_HIP_OK;
    }
    if (T) {
        const dim3 grid = with_side((unsigned)C, T);
        if (N * (inner / 4) <= (size_t)kOpenQuads * T)
            hipLaunchKernelGGL((bn_resident_k<true, false, kOpenQuads>), grid, dim3(T), 0, stream(), (unsigned)N,
                               (unsigned)C, (unsigned)(inner / 4), 0.0, eps, x, dy, scale, (const float *)nullptr,
                               (const float *)nullptr, (const float *)nullptr, ymask, 0, packed, packed + total,
                               packed + total + C, dx_sum, OpenSum{}, pl, sd);
        else
            hipLaunchKernelGGL((bn_resident_k<true, false, kResQuads>), grid, dim3(T), 0, stream(), (unsigned)N,
                               (unsigned)C, (unsigned)(inner / 4), 0.0, eps, x, dy, scale, (const float *)nullptr,
                               (const float *)nullptr, (const float *)nullptr, ymask, 0, packed, packed + total,
                               packed + total + C, dx_sum, OpenSum{}, pl, sd);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    size_t part_bytes = C * kMaxSlices * 4 * sizeof(float);
    char *ws = (char *)workspace(part_bytes + C * sizeof(CoefG));
    if (!ws) return DOPT_HIP_ERR_OOM;
    float *partial = (float *)ws;
    CoefG *coef = (CoefG *)(ws + part_bytes);
    size_t S;
    if (int rc = launch_partial<true>(N, C, inner, x, dy, ymask, partial, &S)) return rc;
    hipLaunchKernelGGL(bn_grad_finalize_k, dim3((unsigned)ceil_div(C, (size_t)kBlock)), dim3(kBlock), 0, stream(), N, C,
                       inner, S, eps, x, partial, scale, coef, packed + total, packed + total + C);
    DOPT_LAUNCH_CHECK();
    bool vec = (inner & 3) == 0 && aligned16(x) && aligned16(dy) && aligned16(packed) && (!ymask || aligned16(ymask));
    unsigned grid = apply_grid(total, vec);
    bool small = total < 0x7fffffffull;
    if (small) {
        if (vec)
            hipLaunchKernelGGL((bn_grad_apply_k<unsigned, true>), dim3(grid), dim3(kBlock), 0, stream(), (unsigned)total,
                               (unsigned)C, (unsigned)inner, dy, ymask, x, coef, packed);
        else
            hipLaunchKernelGGL((bn_grad_apply_k<unsigned, false>), dim3(grid), dim3(kBlock), 0, stream(),
                               (unsigned)total, (unsigned)C, (unsigned)inner, dy, ymask, x, coef, packed);
    } else {
        if (vec)
            hipLaunchKernelGGL((bn_grad_apply_k<size_t, true>), dim3(grid), dim3(kBlock), 0, stream(), total, C, inner,
                               dy, ymask, x, coef, packed);
        else
            hipLaunchKernelGGL((bn_grad_apply_k<size_t, false>), dim3(grid), dim3(kBlock), 0, stream(), total, C, inner,
                               dy, ymask, x, coef, packed);
    }
    DOPT_LAUNCH_CHECK();
    if (dx_sum) return dopt_hip_bias_bwd(N, C, inner, packed, dx_sum);  // large channels: a pass of its own
    return DOPT_HIP_OK;
}

}  // namespace

namespace dopt {

// Called by the library's synchronisation points once the queues are idle: reports a cluster kernel
// whose blocks gave up waiting for each other, and puts the counters back to zero.
int bn_cluster_poll()
{
    if (!g_cluster_unchecked) return DOPT_HIP_OK;
    g_cluster_unchecked = false;
    ClusterMem cm;
    if (int rc = cluster_mem(&cm)) return rc;
    int err = 0;
    DOPT_HIP_CHECK(hipMemcpy(&err, cm.error, sizeof(int), hipMemcpyDeviceToHost));
    if (!err) return DOPT_HIP_OK;
    DOPT_HIP_CHECK(hipMemset(cm.error, 0, sizeof(int)));
    DOPT_HIP_CHECK(hipMemset(cm.rec, 0xff, sizeof(unsigned long long) * kClusterRecs * 4));
    DOPT_HIP_CHECK(hipMemset(cm.depart, 0, kClusterChannels * sizeof(unsigned)));
    DOPT_HIP_CHECK(hipMemset(cm.sdx, 0, kClusterRecs * sizeof(unsigned long long)));
    return fail(DOPT_HIP_ERR_RUNTIME, "batch norm: blocks sharing a channel did not meet within the wait limit; the "
                                      "results of batch-norm calls since the last synchronisation are invalid");
}

unsigned long bn_cluster_launches() { return g_cluster_launches; }
void bn_cluster_mark_unchecked() { g_cluster_unchecked = true; }
bool bn_cluster_pending() { return g_cluster_unchecked; }

int bn_device_setup()
{
    int dev = -1;
    DOPT_HIP_CHECK(hipGetDevice(&dev));
    DOPT_REQUIRE(dev >= 0 && dev < 64, "batch norm: device index %d out of range", dev);
    if (g_cluster_ready[dev]) return DOPT_HIP_OK;
    ClusterMem m;
    DOPT_HIP_CHECK(hipGetSymbolAddress((void **)&m.rec, HIP_SYMBOL(g_cl_rec)));
    DOPT_HIP_CHECK(hipGetSymbolAddress((void **)&m.sdx, HIP_SYMBOL(g_cl_sdx)));
    DOPT_HIP_CHECK(hipGetSymbolAddress((void **)&m.depart, HIP_SYMBOL(g_cl_depart)));
    DOPT_HIP_CHECK(hipGetSymbolAddress((void **)&m.error, HIP_SYMBOL(g_cl_error)));
    // "nothing there" is all-ones (the loader zero-fills); once per device, before any launch
    DOPT_HIP_CHECK(hipMemset(m.rec, 0xff, sizeof(unsigned long long) * kClusterRecs * 4));
    DOPT_HIP_CHECK(hipDeviceSynchronize());
    g_cluster_mem[dev] = m;
    g_cluster_ready[dev] = true;
    return DOPT_HIP_OK;
}

}  // namespace dopt

extern "C" {

int dopt_hip_bn_wait_limit(unsigned polls)
{
    g_cluster_spin_limit = polls;
    return DOPT_HIP_OK;
}

int dopt_hip_bn_train(size_t N, size_t C, size_t inner, double momentum, const float *x, const float *scale,
                      const float *bias, const float *run_mean, const float *run_var, float *packed)
{
    return bn_train_impl(N, C, inner, momentum, x, scale, bias, run_mean, run_var, packed, 0, "dopt_hip_bn_train");
}

int dopt_hip_bn_train_relu(size_t N, size_t C, size_t inner, double momentum, const float *x, const float *scale,
                           const float *bias, const float *run_mean, const float *run_var, float *packed)
{
    return bn_train_impl(N, C, inner, momentum, x, scale, bias, run_mean, run_var, packed, 1, "dopt_hip_bn_train_relu");
}

int dopt_hip_bn_grad(size_t N, size_t C, size_t inner, const float *dy, const float *x, const float *scale,
                     float *packed)
{
    return bn_grad_impl(N, C, inner, dy, nullptr, x, scale, packed, nullptr, "dopt_hip_bn_grad");
}

int dopt_hip_bn_grad_relu(size_t N, size_t C, size_t inner, const float *dy, const float *y, const float *x,
                          const float *scale, float *packed)
{
    DOPT_REQUIRE(y != nullptr, "dopt_hip_bn_grad_relu: null argument");
    return bn_grad_impl(N, C, inner, dy, y, x, scale, packed, nullptr, "dopt_hip_bn_grad_relu");
}

int dopt_hip_bn_train_open(size_t N, size_t C, size_t inner, double momentum, const dopt_hip_split_sum *x_open,
                           const float *scale, const float *bias, const float *run_mean, const float *run_var,
                           float *packed, int relu)
{
    DOPT_REQUIRE(x_open && x_open->value, "dopt_hip_bn_train_open: null argument");
    return bn_train_impl(N, C, inner, momentum, x_open->value, scale, bias, run_mean, run_var, packed, relu != 0,
                         "dopt_hip_bn_train_open", x_open);
}

int dopt_hip_bn_grad_open(size_t N, size_t C, size_t inner, const dopt_hip_split_sum *dy_open, int keep_dy,
                          const float *y, const float *x, const float *scale, float *packed, float *dx_sum)
{
    DOPT_REQUIRE(dy_open && dy_open->value, "dopt_hip_bn_grad_open: null argument");
    return bn_grad_impl(N, C, inner, dy_open->value, y, x, scale, packed, dx_sum, "dopt_hip_bn_grad_open", dy_open,
                        keep_dy != 0);
}

int dopt_hip_bn_train_pool(size_t N, size_t C, size_t H, size_t W, double momentum, const float *x,
                           const dopt_hip_split_sum *x_open, const float *scale, const float *bias,
                           const float *run_mean, const float *run_var, float *packed, int relu, float *pooled)
{
    DOPT_REQUIRE(pooled != nullptr && (x_open ? x_open->value != nullptr : x != nullptr), "dopt_hip_bn_train_pool: null argument");
    DOPT_REQUIRE((H & 1) == 0 && (W & 1) == 0, "dopt_hip_bn_train_pool: images of %zu x %zu do not split into 2 x 2 windows", H, W);
    const PoolArg pa{H, W, pooled, nullptr};
    return bn_train_impl(N, C, H * W, momentum, x_open ? x_open->value : x, scale, bias, run_mean, run_var, packed, relu != 0,
                         "dopt_hip_bn_train_pool", x_open, &pa);
}

int dopt_hip_bn_grad_pool(size_t N, size_t C, size_t H, size_t W, const float *dpooled, const float *y, const float *x,
                          const float *scale, float *packed, float *dx_sum)
{
    DOPT_REQUIRE(dpooled != nullptr && y != nullptr, "dopt_hip_bn_grad_pool: null argument");
    DOPT_REQUIRE((H & 1) == 0 && (W & 1) == 0, "dopt_hip_bn_grad_pool: images of %zu x %zu do not split into 2 x 2 windows", H, W);
    const PoolArg pa{H, W, nullptr, dpooled};
    return bn_grad_impl(N, C, H * W, nullptr, y, x, scale, packed, dx_sum, "dopt_hip_bn_grad_pool", nullptr, true, &pa);
}

int dopt_hip_bn_grad_side(size_t N, size_t C, size_t H, size_t W, const float *dy, const dopt_hip_split_sum *dy_open,
                          int keep_dy, const float *dpooled, const dopt_hip_split_sum *dpooled_open, const float *y,
                          const float *x, const float *scale, float *packed, float *dx_sum, const dopt_hip_split_sum *side)
{
    const char *who = "dopt_hip_bn_grad_side";
    DOPT_REQUIRE((dy != nullptr) + (dy_open != nullptr) + (dpooled != nullptr) == 1,
                 "%s: exactly one of dy, dy_open and dpooled says where the incoming gradient is", who);
    DOPT_REQUIRE(!dpooled_open || dpooled, "%s: dpooled_open without dpooled", who);
    if (dpooled) {
        DOPT_REQUIRE(y != nullptr, "%s: the pooled form needs y", who);
        DOPT_REQUIRE((H & 1) == 0 && (W & 1) == 0, "%s: images of %zu x %zu do not split into 2 x 2 windows", who, H, W);
        DOPT_REQUIRE(!dpooled_open || dpooled_open->value == dpooled, "%s: dpooled is not the open value", who);
        PoolArg pa{H, W, nullptr, dpooled};
        pa.dopen = dpooled_open;
        pa.keep = keep_dy != 0;
        return bn_grad_impl(N, C, H * W, nullptr, y, x, scale, packed, dx_sum, who, nullptr, true, &pa, side);
    }
    if (dy_open) {
        DOPT_REQUIRE(dy_open->value != nullptr, "%s: null argument", who);
        return bn_grad_impl(N, C, H * W, dy_open->value, y, x, scale, packed, dx_sum, who, dy_open, keep_dy != 0, nullptr, side);
    }
    return bn_grad_impl(N, C, H * W, dy, y, x, scale, packed, dx_sum, who, nullptr, true, nullptr, side);
}

int dopt_hip_bn_grad_fused(size_t N, size_t C, size_t inner, const float *dy, const float *y, const float *x,
                           const float *scale, float *packed, float *dx_sum)
{
    return bn_grad_impl(N, C, inner, dy, y, x, scale, packed, dx_sum, "dopt_hip_bn_grad_fused");
}

int dopt_hip_bn_infer(size_t N, size_t C, size_t inner, const float *x, const float *scale, const float *bias,
                      const float *mean, const float *var, float *y)
{
    size_t total = N * C * inner;
    if (total == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && scale && bias && mean && var && y, "dopt_hip_bn_infer: null argument");
    DOPT_ENSURE_INIT();
    if ((inner & 3) == 0 && inner >= 256 && aligned16(x) && aligned16(y) && total / 4 < 0xffffffffull && N < (1u << 24) &&
        C <= 0x7fffffffu / kMaxSlices) {
        const size_t S = pick_slices(N, C);
        hipLaunchKernelGGL(bn_infer_chan_k, dim3((unsigned)(C * S)), dim3(kBlock), 0, stream(), (unsigned)N, (unsigned)C,
                           (unsigned)(inner / 4), (unsigned)S, 1e-5 /* cudnn7.d:652 */, x, scale, bias, mean, var, y);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    Coef *coef = (Coef *)workspace(C * sizeof(Coef));
    if (!coef) return DOPT_HIP_ERR_OOM;
    hipLaunchKernelGGL(bn_infer_prepare_k, dim3((unsigned)ceil_div(C, (size_t)kBlock)), dim3(kBlock), 0, stream(), C,
                       1e-5 /* cudnn7.d:652 */, scale, bias, mean, var, coef);
    DOPT_LAUNCH_CHECK();
    return launch_apply(total, C, inner, x, coef, y, 0);
}

}  // extern "C"
