// Bandwidth-bound NN ops (fp32, NCHW): relu, addBias, maxpool, softmax and their gradients.
// Each replaces one cuDNN call of cuda/source/dopt/cuda/nnet/cudnn7.d (cited per entry point in
// include/dopt_hip.h) with a single streaming kernel: every input is read once and every
// output written once, with 128-bit accesses wherever the shapes allow.
#include <cfloat>

#include "common.h"
#include "pool2x2.h"

namespace {

using namespace dopt;

constexpr int kBlock = 256;
constexpr int kUnroll = 4;

unsigned stream_grid(size_t n4)
{
    size_t blocks = ceil_div(n4, (size_t)kBlock * kUnroll);
    size_t cap = (size_t)num_cus() * 8;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

unsigned flat_grid(size_t n)
{
    size_t blocks = ceil_div(n, (size_t)kBlock);
    size_t cap = (size_t)num_cus() * 16;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

// NaN propagates (CUDNN_PROPAGATE_NAN): NaN < 0 is false, so x passes through.
__device__ inline float relu1(float x) { return x < 0.0f ? 0.0f : x; }
__device__ inline float relu_grad1(float dy, float x) { return x > 0.0f ? dy : 0.0f; }

// ---------------------------------------------------------------------------------- relu
template <bool kVec>
__global__ __launch_bounds__(kBlock) void relu_fwd_k(size_t n, const float *x, float *y)
{
    if (kVec) {
        const size_t n4 = n >> 2;
        const float4 *x4 = (const float4 *)x;
        float4 *y4 = (float4 *)y;
        for (size_t base = (size_t)blockIdx.x * (kBlock * kUnroll); base < n4;
             base += (size_t)gridDim.x * (kBlock * kUnroll)) {
            float4 v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4) v[u] = x4[i];
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4) y4[i] = make_float4(relu1(v[u].x), relu1(v[u].y), relu1(v[u].z), relu1(v[u].w));
            }
        }
        if (blockIdx.x == 0) {
            size_t i = (n4 << 2) + threadIdx.x;
            if (i < n) y[i] = relu1(x[i]);
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
            y[i] = relu1(x[i]);
    }
}

template <bool kVec>
__global__ __launch_bounds__(kBlock) void relu_bwd_k(size_t n, const float *dy, const float *x, float *dx)
{
    if (kVec) {
        const size_t n4 = n >> 2;
        const float4 *g4 = (const float4 *)dy;
        const float4 *x4 = (const float4 *)x;
        float4 *o4 = (float4 *)dx;
        for (size_t base = (size_t)blockIdx.x * (kBlock * kUnroll); base < n4;
             base += (size_t)gridDim.x * (kBlock * kUnroll)) {
            float4 g[kUnroll], v[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4) {
                    g[u] = g4[i];
                    v[u] = x4[i];
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4)
                    o4[i] = make_float4(relu_grad1(g[u].x, v[u].x), relu_grad1(g[u].y, v[u].y),
                                        relu_grad1(g[u].z, v[u].z), relu_grad1(g[u].w, v[u].w));
            }
        }
        if (blockIdx.x == 0) {
            size_t i = (n4 << 2) + threadIdx.x;
            if (i < n) dx[i] = relu_grad1(dy[i], x[i]);
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
            dx[i] = relu_grad1(dy[i], x[i]);
    }
}

// ---------------------------------------------------------------------------------- bias
// y[n,c,i] = x[n,c,i] + b[c].  kVec needs inner % 4 == 0 so that a float4 stays inside one channel.
template <bool kVec>
__global__ __launch_bounds__(kBlock) void bias_fwd_k(size_t total, size_t C, size_t inner, const float *x,
                                                      const float *b, float *y)
{
    if (kVec) {
        const size_t n4 = total >> 2, inner4 = inner >> 2;
        const float4 *x4 = (const float4 *)x;
        float4 *y4 = (float4 *)y;
        for (size_t base = (size_t)blockIdx.x * (kBlock * kUnroll); base < n4;
             base += (size_t)gridDim.x * (kBlock * kUnroll)) {
            float4 v[kUnroll];
            float bb[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4) {
                    v[u] = x4[i];
                    bb[u] = b[(i / inner4) % C];
                }
            }
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                size_t i = base + (size_t)u * kBlock + threadIdx.x;
                if (i < n4) y4[i] = make_float4(v[u].x + bb[u], v[u].y + bb[u], v[u].z + bb[u], v[u].w + bb[u]);
            }
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock)
            y[i] = x[i] + b[(i / inner) % C];
    }
}

__device__ inline float block_sum(float v, float *part)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.0f;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kBlock / 64; w++) r += part[w];
    }
    __syncthreads();
    return r;  // valid in thread 0
}

__global__ __launch_bounds__(kBlock) void fill_zero_k(size_t n, float *out)
{
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = 0.0f;
}

// Stage 1 of db[c] = sum_{n,i} dy[n,c,i]: block (c, s) sums images n = s, s + S, ... of channel c with four
// independent 128-bit (or 32-bit) loads in flight per thread.
// (Finishing in the same launch -- the last block of a channel, found by a ticket counter, adds the S
// sums -- was built twice and measured: with device-scope release/acquire per block 41 us, with
// fence-free tagged words 14.3 us, against 9 us for the two launches; the second launch is cheaper
// than 2048 device-scope atomics.)
template <typename V>   // float4: rows of `inner` floats are 16-byte aligned multiples of four; float otherwise
__global__ __launch_bounds__(kBlock) void chan_sum_k(unsigned N, unsigned C, unsigned inner, unsigned S, const float *dy,
                                                      float *partial)
{
    __shared__ float part[kBlock / 64];
    constexpr unsigned kPer = sizeof(V) / sizeof(float);
    const unsigned c = blockIdx.x % C, s = blockIdx.x / C;
    const unsigned row = inner / kPer;                     // V per (image, channel) row
    const unsigned nimg = (N - s + S - 1) / S, tot = nimg * row;
    auto at = [&](unsigned t) -> V {
        const unsigned j = t / row, i = t - j * row;
        return ((const V *)(dy + ((size_t)(s + j * S) * C + c) * inner))[i];
    };
    auto fold = [](const V &v) -> float {
        if constexpr (sizeof(V) == 16) return (v.x + v.y) + (v.z + v.w);
        else return v;
    };
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    unsigned t = threadIdx.x;
    for (; t + 3 * kBlock < tot; t += 4 * kBlock) {
        const V v0 = at(t), v1 = at(t + kBlock), v2 = at(t + 2 * kBlock), v3 = at(t + 3 * kBlock);
        a0 += fold(v0);
        a1 += fold(v1);
        a2 += fold(v2);
        a3 += fold(v3);
    }
    for (; t < tot; t += kBlock) a0 += fold(at(t));
    const float r = block_sum((a0 + a1) + (a2 + a3), part);
    if (threadIdx.x == 0) partial[c * S + s] = r;
}

// Stage 2: fixed-order sum of the S partials of each channel (deterministic, no atomics).
__global__ __launch_bounds__(kBlock) void chan_sum_final_k(size_t C, size_t S, const float *partial, float *db)
{
    size_t c = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (c >= C) return;
    float acc = 0.0f;
    for (size_t s = 0; s < S; s++) acc += partial[c * S + s];
    db[c] = acc;
}

// Variant for small `inner` (dense layers, tiny feature maps): thread t walks (n, i) pairs of channel c.
__global__ __launch_bounds__(kBlock) void bias_bwd_flat_k(size_t N, size_t C, size_t inner, const float *dy,
                                                           float *db)
{
    __shared__ float part[kBlock / 64];
    const size_t c = blockIdx.x;
    const size_t per = N * inner;
    float acc = 0.0f;
    for (size_t j = threadIdx.x; j < per; j += kBlock) {
        size_t n = j / inner, i = j % inner;
        acc += dy[(n * C + c) * inner + i];
    }
    float r = block_sum(acc, part);
    if (threadIdx.x == 0) db[c] = r;
}

// ---------------------------------------------------------------------------------- maxpool
// The comparison chains (dmax, pool2x2, route2x2) live in pool2x2.h: the batch-norm kernels share them.

// 2x2 windows, W % 4 == 0, 16-byte aligned: one thread makes two adjacent outputs from two float4 rows.
__global__ __launch_bounds__(kBlock) void maxpool2x2_fwd_k(size_t maps, size_t H, size_t W, const float *x, float *y)
{
    const size_t P = H >> 1, Q2 = W >> 2;  // output rows, output column PAIRS
    const size_t total = maps * P * Q2;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t q2 = idx % Q2, t = idx / Q2;
        size_t p = t % P, m = t / P;
        const float4 *r0 = (const float4 *)(x + (m * H + 2 * p) * W) + q2;
        const float4 *r1 = (const float4 *)(x + (m * H + 2 * p + 1) * W) + q2;
        float4 a = *r0, b = *r1;
        float o0 = pool2x2(a.x, a.y, b.x, b.y);
        float o1 = pool2x2(a.z, a.w, b.z, b.w);
        ((float2 *)(y + (m * P + p) * (W >> 1)))[q2] = make_float2(o0, o1);
    }
}

__global__ __launch_bounds__(kBlock) void maxpool_fwd_k(size_t maps, size_t H, size_t W, size_t ph, size_t pw,
                                                         const float *x, float *y)
{
    const size_t P = H / ph, Q = W / pw;
    const size_t total = maps * P * Q;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t q = idx % Q, t = idx / Q;
        size_t p = t % P, m = t / P;
        const float *img = x + m * H * W;
        float acc = -FLT_MAX;
        for (size_t j = 0; j < ph; j++)
            for (size_t i = 0; i < pw; i++) acc = dmax(acc, img[(p * ph + j) * W + q * pw + i]);
        y[idx] = acc;
    }
}

// 2x2, H even, W % 4 == 0, aligned: a thread owns two adjacent windows = a float4 of each of two rows.
__global__ __launch_bounds__(kBlock) void maxpool2x2_bwd_k(size_t maps, size_t H, size_t W, const float *dy,
                                                            const float *x, float *dx)
{
    const size_t P = H >> 1, Q2 = W >> 2;
    const size_t total = maps * P * Q2;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t q2 = idx % Q2, t = idx / Q2;
        size_t p = t % P, m = t / P;
        size_t row0 = (m * H + 2 * p) * W, row1 = row0 + W;
        float4 a = ((const float4 *)(x + row0))[q2], b = ((const float4 *)(x + row1))[q2];
        float2 g = ((const float2 *)(dy + (m * P + p) * (W >> 1)))[q2];
        float4 oa, ob;
        route2x2(a.x, a.y, b.x, b.y, g.x, oa.x, oa.y, ob.x, ob.y);
        route2x2(a.z, a.w, b.z, b.w, g.y, oa.z, oa.w, ob.z, ob.w);
        ((float4 *)(dx + row0))[q2] = oa;
        ((float4 *)(dx + row1))[q2] = ob;
    }
}

// General windows: one thread per INPUT element; rows/columns beyond the last full window get 0.
__global__ __launch_bounds__(kBlock) void maxpool_bwd_k(size_t maps, size_t H, size_t W, size_t ph, size_t pw,
                                                         const float *dy, const float *x, float *dx)
{
    const size_t P = H / ph, Q = W / pw;
    const size_t total = maps * H * W;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t w = idx % W, t = idx / W;
        size_t h = t % H, m = t / H;
        size_t p = h / ph, q = w / pw;
        float out = 0.0f;
        if (p < P && q < Q) {
            const float *img = x + m * H * W;
            size_t best = (p * ph) * W + q * pw;
            float bv = -FLT_MAX;   // the forward pass's own chain of tests
            for (size_t j = 0; j < ph; j++)
                for (size_t i = 0; i < pw; i++) {
                    size_t e = (p * ph + j) * W + q * pw + i;
                    float v = img[e];
                    if (bv < v) { bv = v; best = e; }
                }
            if (best == h * W + w) out = dy[(m * P + p) * Q + q];
        }
        dx[idx] = out;
    }
}

// ---------------------------------------------------------------------------------- softmax
// One thread per (n, i) lane, channel loop in the order of cpu/nnet.d:129-166: max, exp and
// running fp32 sum, divide.
__global__ __launch_bounds__(kBlock) void softmax_fwd_k(size_t N, size_t C, size_t inner, const float *x, float *y)
{
    const size_t total = N * inner;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t n = idx / inner, i = idx % inner;
        const float *px = x + n * C * inner + i;
        float *py = y + n * C * inner + i;
        float m = -FLT_MAX;
        for (size_t c = 0; c < C; c++) m = dmax(m, px[c * inner]);
        float s = 0.0f;
        for (size_t c = 0; c < C; c++) {
            float pot = expf(px[c * inner] - m);
            s += pot;
            py[c * inner] = pot;
        }
        for (size_t c = 0; c < C; c++) py[c * inner] = py[c * inner] / s;
    }
}

// Rows of at least 64 contiguous channels (inner == 1): one wavefront per row, lanes stride along
// the channels, maximum / sum / dot product folded with wavefront shuffles.  Sums are tree-ordered
// here (the lane-per-row kernels sum in channel order).
__device__ inline float wave_allsum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__global__ __launch_bounds__(kBlock) void softmax_rows_fwd_k(size_t N, size_t C, const float *x, float *y)
{
    const size_t row = (size_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (row >= N) return;
    const int lane = threadIdx.x & 63;
    const float *px = x + row * C;
    float *py = y + row * C;
    float m = -FLT_MAX;
    for (size_t c = lane; c < C; c += 64) m = dmax(m, px[c]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = dmax(m, __shfl_xor(m, off, 64));
    float s = 0.0f;
    for (size_t c = lane; c < C; c += 64) {
        const float pot = expf(px[c] - m);
        s += pot;
        py[c] = pot;
    }
    s = wave_allsum(s);
    for (size_t c = lane; c < C; c += 64) py[c] = py[c] / s;
}

// Rows of at most 1024 values whose length is a multiple of four stay in registers: G lanes share a
// row (64 / G rows per wavefront), each lane holds up to four quads, the row is read once and
// written once.
template <int G>
__device__ __forceinline__ float group_max(float v)
{
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v = dmax(v, __shfl_xor(v, off, 64));
    return v;
}

template <int G>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int G, int Q>   // G lanes share a row, Q quads per lane (G * Q >= C / 4)
__global__ __launch_bounds__(kBlock) void softmax_reg_fwd_k(size_t N, uint32_t C4, const float4 *x, float4 *y)
{
    const size_t row = ((size_t)blockIdx.x * kBlock + threadIdx.x) / G;
    const uint32_t lig = threadIdx.x % G;
    const bool live = row < N;                    // dead rows still take part in the shuffles
    const float4 *px = x + (live ? row : 0) * C4;
    float v[4 * Q];
#pragma unroll
    for (int k = 0; k < Q; k++) {
        const uint32_t c = lig + G * k;
        const float4 q = px[c < C4 ? c : 0];
        const bool in = c < C4;
        v[4 * k + 0] = in ? q.x : -FLT_MAX;
        v[4 * k + 1] = in ? q.y : -FLT_MAX;
        v[4 * k + 2] = in ? q.z : -FLT_MAX;
        v[4 * k + 3] = in ? q.w : -FLT_MAX;
    }
    float m = v[0];
#pragma unroll
    for (int i = 1; i < 4 * Q; i++) m = dmax(m, v[i]);
    m = group_max<G>(m);
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < Q; k++) {
        const bool in = lig + G * k < C4;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[4 * k + j] = in ? expf(v[4 * k + j] - m) : 0.0f;
            s += v[4 * k + j];
        }
    }
    s = group_sum<G>(s);
    if (!live) return;
    float4 *py = y + row * C4;
#pragma unroll
    for (int k = 0; k < Q; k++) {
        const uint32_t c = lig + G * k;
        if (c < C4) py[c] = make_float4(v[4 * k] / s, v[4 * k + 1] / s, v[4 * k + 2] / s, v[4 * k + 3] / s);
    }
}

template <int G, int Q>
__global__ __launch_bounds__(kBlock) void softmax_reg_bwd_k(size_t N, uint32_t C4, const float4 *dy, const float4 *y,
                                                             float4 *dx)
{
    const size_t row = ((size_t)blockIdx.x * kBlock + threadIdx.x) / G;
    const uint32_t lig = threadIdx.x % G;
    const bool live = row < N;
    const size_t base = (live ? row : 0) * C4;
    float g[4 * Q], p[4 * Q];
    float dot = 0.0f;
#pragma unroll
    for (int k = 0; k < Q; k++) {
        const uint32_t c = lig + G * k;
        const bool in = c < C4;
        const float4 a = dy[base + (in ? c : 0)], b = y[base + (in ? c : 0)];
        g[4 * k + 0] = a.x, g[4 * k + 1] = a.y, g[4 * k + 2] = a.z, g[4 * k + 3] = a.w;
        p[4 * k + 0] = b.x, p[4 * k + 1] = b.y, p[4 * k + 2] = b.z, p[4 * k + 3] = b.w;
        if (in) dot += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
    }
    dot = group_sum<G>(dot);
    if (!live) return;
#pragma unroll
    for (int k = 0; k < Q; k++) {
        const uint32_t c = lig + G * k;
        if (c < C4)
            dx[base + c] = make_float4(p[4 * k] * (g[4 * k] - dot), p[4 * k + 1] * (g[4 * k + 1] - dot),
                                       p[4 * k + 2] * (g[4 * k + 2] - dot), p[4 * k + 3] * (g[4 * k + 3] - dot));
    }
}

// the lanes a row of C4 quads is shared by, or 0 when the register kernels do not take it
int softmax_group(size_t C, size_t inner, const void *a, const void *b, const void *c)
{
    if (inner != 1 || C % 4 != 0 || C < 64 || C > 1024 || !aligned16(a) || !aligned16(b) || !aligned16(c)) return 0;
    const size_t C4 = C / 4;
    return C4 <= 16 ? 16 : (C4 <= 32 ? 32 : 64);
}

__global__ __launch_bounds__(kBlock) void softmax_rows_bwd_k(size_t N, size_t C, const float *dy, const float *y,
                                                              float *dx)
{
    const size_t row = (size_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (row >= N) return;
    const int lane = threadIdx.x & 63;
    const size_t base = row * C;
    float dot = 0.0f;
    for (size_t c = lane; c < C; c += 64) dot += dy[base + c] * y[base + c];
    dot = wave_allsum(dot);
    for (size_t c = lane; c < C; c += 64) dx[base + c] = y[base + c] * (dy[base + c] - dot);
}

__global__ __launch_bounds__(kBlock) void softmax_bwd_k(size_t N, size_t C, size_t inner, const float *dy,
                                                         const float *y, float *dx)
{
    const size_t total = N * inner;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t n = idx / inner, i = idx % inner;
        size_t base = n * C * inner + i;
        float dot = 0.0f;
        for (size_t c = 0; c < C; c++) dot += dy[base + c * inner] * y[base + c * inner];
        for (size_t c = 0; c < C; c++) dx[base + c * inner] = y[base + c * inner] * (dy[base + c * inner] - dot);
    }
}

// ---------------------------------------------------------------------------------- uniform
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): a
// counter-based generator, so element i of call c depends only on (seed, c, i) -- no generator
// state in device memory, any launch shape gives the same stream.  A 128-bit counter block
// yields four 32-bit words; word -> float in (0, 1] as curandGenerateUniform documents its range
// (cuda/random.d:74; the CPU kernel shifts D's [0, 1) by epsilon for the same reason,
// cpu/random.d:24).
__device__ inline void philox_round(uint32_t (&c)[4], uint32_t k0, uint32_t k1)
{
    const uint32_t lo0 = 0xD2511F53u * c[0], hi0 = __umulhi(0xD2511F53u, c[0]);
    const uint32_t lo1 = 0xCD9E8D57u * c[2], hi1 = __umulhi(0xCD9E8D57u, c[2]);
    const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
    c[0] = n0;
    c[1] = lo1;
    c[2] = n2;
    c[3] = lo0;
}

__device__ inline void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1)
{
#pragma unroll
    for (int r = 0; r < 10; r++) {
        philox_round(c, k0, k1);
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

__device__ inline float u01(uint32_t w) { return (float)((w >> 8) + 1u) * 5.9604644775390625e-8f; }  // (0, 1], 2^-24 steps

// Block b of four outputs uses counter (b, call_lo, call_hi, 0) and key (seed_lo, seed_hi).
__global__ __launch_bounds__(kBlock) void uniform_k(size_t n, uint64_t seed, uint64_t call, float *out, uint32_t *raw)
{
    const size_t nb = (n + 3) / 4;
    for (size_t b = (size_t)blockIdx.x * kBlock + threadIdx.x; b < nb; b += (size_t)gridDim.x * kBlock) {
        uint32_t c[4] = {(uint32_t)b, (uint32_t)call, (uint32_t)(call >> 32), (uint32_t)(b >> 32)};
        philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const size_t i = b * 4 + j;
            if (i < n) {
                if (raw) raw[i] = c[j];
                else out[i] = u01(c[j]);
            }
        }
    }
}

}  // namespace

extern "C" {

int dopt_hip_relu_fwd(size_t n, const float *x, float *y)
{
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && y, "dopt_hip_relu_fwd: null argument");
    DOPT_ENSURE_INIT();
    if (aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(relu_fwd_k<true>, dim3(stream_grid(n / 4)), dim3(kBlock), 0, stream(), n, x, y);
    else
        hipLaunchKernelGGL(relu_fwd_k<false>, dim3(flat_grid(n)), dim3(kBlock), 0, stream(), n, x, y);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_relu_bwd(size_t n, const float *dy, const float *x, float *dx)
{
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dy && x && dx, "dopt_hip_relu_bwd: null argument");
    DOPT_ENSURE_INIT();
    if (aligned16(dy) && aligned16(x) && aligned16(dx))
        hipLaunchKernelGGL(relu_bwd_k<true>, dim3(stream_grid(n / 4)), dim3(kBlock), 0, stream(), n, dy, x, dx);
    else
        hipLaunchKernelGGL(relu_bwd_k<false>, dim3(flat_grid(n)), dim3(kBlock), 0, stream(), n, dy, x, dx);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_bias_fwd(size_t N, size_t C, size_t inner, const float *x, const float *b, float *y)
{
    size_t total = N * C * inner;
    if (total == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && b && y, "dopt_hip_bias_fwd: null argument");
    DOPT_ENSURE_INIT();
    if ((inner & 3) == 0 && aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(bias_fwd_k<true>, dim3(stream_grid(total / 4)), dim3(kBlock), 0, stream(), total, C, inner,
                           x, b, y);
    else
        hipLaunchKernelGGL(bias_fwd_k<false>, dim3(flat_grid(total)), dim3(kBlock), 0, stream(), total, C, inner, x,
                           b, y);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// How many image slices per channel: enough (channel, slice) blocks to fill the machine.
static size_t bias_bwd_slices(size_t N, size_t C)
{
    size_t S = ceil_div((size_t)num_cus() * 8, C);
    if (S > N) S = N;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    return S;
}

static constexpr int kMaxDevices = 64;

// The sliced sum; `partial` holds C * S floats, every one of which stage 1 writes before stage 2 reads it
// (nothing has to be cleared).
static int chan_sum_launch(size_t N, size_t C, size_t inner, size_t S, const float *dy, float *partial, float *db)
{
    const unsigned grid = (unsigned)(C * S);
    if ((inner & 3) == 0 && aligned16(dy))
        hipLaunchKernelGGL((chan_sum_k<float4>), dim3(grid), dim3(kBlock), 0, stream(), (unsigned)N, (unsigned)C, (unsigned)inner,
                           (unsigned)S, dy, partial);
    else
        hipLaunchKernelGGL((chan_sum_k<float>), dim3(grid), dim3(kBlock), 0, stream(), (unsigned)N, (unsigned)C, (unsigned)inner,
                           (unsigned)S, dy, partial);
    DOPT_LAUNCH_CHECK();
    hipLaunchKernelGGL(chan_sum_final_k, dim3((unsigned)ceil_div(C, (size_t)kBlock)), dim3(kBlock), 0, stream(), C, S, partial, db);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// Whether the sliced sum takes the shape (32-bit indexing inside a slice).
static bool chan_sum_takes(size_t N, size_t C, size_t inner)
{
    return inner >= 256 && N < (1u << 24) && inner < (1u << 24) && N * inner < (1ull << 32) && C <= 0x7fffffffu / 64;
}

int dopt_hip_bias_bwd(size_t N, size_t C, size_t inner, const float *dy, float *db)
{
    if (C == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(db && (N * inner == 0 || dy), "dopt_hip_bias_bwd: null argument");
    DOPT_ENSURE_INIT();
    if (N * inner == 0) return dopt_hip_memset(db, 0, C * sizeof(float));
    DOPT_REQUIRE(C <= 0x7fffffffu / 64, "dopt_hip_bias_bwd: too many channels");
    if (!chan_sum_takes(N, C, inner)) {
        hipLaunchKernelGGL(bias_bwd_flat_k, dim3((unsigned)C), dim3(kBlock), 0, stream(), N, C, inner, dy, db);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    const size_t S = bias_bwd_slices(N, C);
    float *partial = (float *)workspace(C * S * sizeof(float));
    if (!partial) return DOPT_HIP_ERR_OOM;
    return chan_sum_launch(N, C, inner, S, dy, partial, db);
}

// ---- the same sum for callers that must not allocate
// The per-(channel, slice) partial sums live in this array instead of the library's grown-on-demand
// workspace, and the call sets nothing up: the array's address on the device is taken by dopt_hip_init
// (nn_device_setup), which is also what makes the runtime load this file's code object, array included.
// Every device the library runs on holds its own copy at its own address until the process ends; host
// code only ever uses the address hipGetSymbolAddress reported for that device.
static constexpr size_t kBiasScratchFloats = 65536;   // 256 KiB
static __device__ __align__(256) float scratch[kBiasScratchFloats];
static float *g_scratch_ptr[kMaxDevices];             // per device; set by dopt_hip_init

int dopt_hip_bias_bwd_noalloc(size_t N, size_t C, size_t inner, const float *dy, float *db)
{
    if (C == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(db && (N * inner == 0 || dy), "dopt_hip_bias_bwd_noalloc: null argument");
    DOPT_REQUIRE(is_initialised(), "dopt_hip_bias_bwd_noalloc: call dopt_hip_init first (this entry point sets nothing up)");
    DOPT_REQUIRE(C <= 0x7fffffffu / 64, "dopt_hip_bias_bwd_noalloc: too many channels");
    if (N * inner == 0) {   // a fill kernel, not a memset node: callers may be recording a graph
        hipLaunchKernelGGL(fill_zero_k, dim3((unsigned)ceil_div(C, (size_t)kBlock)), dim3(kBlock), 0, stream(), C, db);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    const size_t S = bias_bwd_slices(N, C);
    if (inner < 256) {      // short rows: one launch, no partial sums, same kernel as dopt_hip_bias_bwd
        hipLaunchKernelGGL(bias_bwd_flat_k, dim3((unsigned)C), dim3(kBlock), 0, stream(), N, C, inner, dy, db);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    DOPT_REQUIRE(C * S <= kBiasScratchFloats && chan_sum_takes(N, C, inner),
                 "dopt_hip_bias_bwd_noalloc: %zu channels x %zu slices exceed the built-in scratch of %zu partial sums; "
                 "use dopt_hip_bias_bwd", C, S, kBiasScratchFloats);
    int dev = -1;
    DOPT_HIP_CHECK(hipGetDevice(&dev));
    DOPT_REQUIRE(dev >= 0 && dev < kMaxDevices, "dopt_hip_bias_bwd_noalloc: device index %d out of range", dev);
    DOPT_REQUIRE(g_scratch_ptr[dev] != nullptr, "dopt_hip_bias_bwd_noalloc: device %d was not set up by dopt_hip_init", dev);
    return chan_sum_launch(N, C, inner, S, dy, g_scratch_ptr[dev], db);
}

int dopt_hip_maxpool_fwd(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw, const float *x, float *y)
{
    DOPT_REQUIRE(ph > 0 && pw > 0, "dopt_hip_maxpool_fwd: pool dims must be positive");
    size_t maps = N * C, P = H / ph, Q = W / pw;
    if (maps * P * Q == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && y, "dopt_hip_maxpool_fwd: null argument");
    DOPT_ENSURE_INIT();
    if (ph == 2 && pw == 2 && (H & 1) == 0 && (W & 3) == 0 && aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(maxpool2x2_fwd_k, dim3(flat_grid(maps * P * (W / 4))), dim3(kBlock), 0, stream(), maps, H, W,
                           x, y);
    else
        hipLaunchKernelGGL(maxpool_fwd_k, dim3(flat_grid(maps * P * Q)), dim3(kBlock), 0, stream(), maps, H, W, ph, pw,
                           x, y);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_maxpool_bwd(size_t N, size_t C, size_t H, size_t W, size_t ph, size_t pw, const float *dy,
                         const float *x, float *dx)
{
    DOPT_REQUIRE(ph > 0 && pw > 0, "dopt_hip_maxpool_bwd: pool dims must be positive");
    size_t maps = N * C;
    if (maps * H * W == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && dx && ((H / ph) * (W / pw) == 0 || dy), "dopt_hip_maxpool_bwd: null argument");
    DOPT_ENSURE_INIT();
    if (ph == 2 && pw == 2 && (H & 1) == 0 && (W & 3) == 0 && aligned16(x) && aligned16(dx) && aligned16(dy))
        hipLaunchKernelGGL(maxpool2x2_bwd_k, dim3(flat_grid(maps * (H / 2) * (W / 4))), dim3(kBlock), 0, stream(), maps,
                           H, W, dy, x, dx);
    else
        hipLaunchKernelGGL(maxpool_bwd_k, dim3(flat_grid(maps * H * W)), dim3(kBlock), 0, stream(), maps, H, W, ph, pw,
                           dy, x, dx);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_softmax_fwd(size_t N, size_t C, size_t inner, const float *x, float *y)
{
    if (N * C * inner == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(x && y, "dopt_hip_softmax_fwd: null argument");
    DOPT_ENSURE_INIT();
    if (const int G = softmax_group(C, inner, x, y, y)) {
        const dim3 grid((unsigned)ceil_div(N * G, (size_t)kBlock)), block(kBlock);
        const uint32_t C4 = (uint32_t)(C / 4);
        // quads per lane: one up to 256 classes, two or four above (no work on lanes' absent quads)
#define DOPT_SOFTMAX_FWD(GV, QV) \
    hipLaunchKernelGGL((softmax_reg_fwd_k<GV, QV>), grid, block, 0, stream(), N, C4, (const float4 *)x, (float4 *)y)
        if (G == 16) DOPT_SOFTMAX_FWD(16, 1);
        else if (G == 32) DOPT_SOFTMAX_FWD(32, 1);
        else if (C4 <= 64) DOPT_SOFTMAX_FWD(64, 1);
        else if (C4 <= 128) DOPT_SOFTMAX_FWD(64, 2);
        else DOPT_SOFTMAX_FWD(64, 4);
#undef DOPT_SOFTMAX_FWD
    } else if (inner == 1 && C >= 64)
        hipLaunchKernelGGL(softmax_rows_fwd_k, dim3((unsigned)ceil_div(N, (size_t)(kBlock / 64))), dim3(kBlock), 0, stream(),
                           N, C, x, y);
    else
        hipLaunchKernelGGL(softmax_fwd_k, dim3(flat_grid(N * inner)), dim3(kBlock), 0, stream(), N, C, inner, x, y);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_softmax_bwd(size_t N, size_t C, size_t inner, const float *dy, const float *y, float *dx)
{
    if (N * C * inner == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(dy && y && dx, "dopt_hip_softmax_bwd: null argument");
    DOPT_ENSURE_INIT();
    if (const int G = softmax_group(C, inner, dy, y, dx)) {
        const dim3 grid((unsigned)ceil_div(N * G, (size_t)kBlock)), block(kBlock);
        const uint32_t C4 = (uint32_t)(C / 4);
#define DOPT_SOFTMAX_BWD(GV, QV)                                                                                  \
    hipLaunchKernelGGL((softmax_reg_bwd_k<GV, QV>), grid, block, 0, stream(), N, C4, (const float4 *)dy, (const float4 *)y, \
                       (float4 *)dx)
        if (G == 16) DOPT_SOFTMAX_BWD(16, 1);
        else if (G == 32) DOPT_SOFTMAX_BWD(32, 1);
        else if (C4 <= 64) DOPT_SOFTMAX_BWD(64, 1);
        else if (C4 <= 128) DOPT_SOFTMAX_BWD(64, 2);
        else DOPT_SOFTMAX_BWD(64, 4);
#undef DOPT_SOFTMAX_BWD
    } else if (inner == 1 && C >= 64)
        hipLaunchKernelGGL(softmax_rows_bwd_k, dim3((unsigned)ceil_div(N, (size_t)(kBlock / 64))), dim3(kBlock), 0, stream(),
                           N, C, dy, y, dx);
    else
        hipLaunchKernelGGL(softmax_bwd_k, dim3(flat_grid(N * inner)), dim3(kBlock), 0, stream(), N, C, inner, dy, y, dx);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_uniform(uint64_t seed, uint64_t call, size_t n, float *out)
{
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(out != nullptr, "dopt_hip_uniform: null argument");
    DOPT_ENSURE_INIT();
    hipLaunchKernelGGL(uniform_k, dim3(flat_grid((n + 3) / 4)), dim3(kBlock), 0, stream(), n, seed, call, out,
                       (uint32_t *)nullptr);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_philox_raw(uint64_t seed, uint64_t call, size_t n, uint32_t *out)
{
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(out != nullptr, "dopt_hip_philox_raw: null argument");
    DOPT_ENSURE_INIT();
    hipLaunchKernelGGL(uniform_k, dim3(flat_grid((n + 3) / 4)), dim3(kBlock), 0, stream(), n, seed, call,
                       (float *)nullptr, out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

}  // extern "C"

namespace dopt {

// out[c] = sum over n and i of in[n][c][i] for rtc_ops.cpp's `sum` over the axes around one kept run of
// axes; false (nothing launched) when the shape is not the one-launch kernel's.
bool channel_sum(size_t N, size_t C, size_t inner, const float *in, float *out, int *rc)
{
    if (!chan_sum_takes(N, C, inner)) return false;
    const size_t S = bias_bwd_slices(N, C);
    float *partial = (float *)workspace(C * S * sizeof(float));
    *rc = partial ? chan_sum_launch(N, C, inner, S, in, partial, out) : DOPT_HIP_ERR_OOM;
    return true;
}

int nn_device_setup()
{
    int dev = -1;
    DOPT_HIP_CHECK(hipGetDevice(&dev));
    DOPT_REQUIRE(dev >= 0 && dev < kMaxDevices, "dopt_hip_init: device index %d out of range", dev);
    if (g_scratch_ptr[dev]) return DOPT_HIP_OK;
    float *p = nullptr;
    DOPT_HIP_CHECK(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    DOPT_REQUIRE(p != nullptr, "dopt_hip_init: the scratch array of dopt_hip_bias_bwd_noalloc has no device address");
    g_scratch_ptr[dev] = p;
    return DOPT_HIP_OK;
}

}  // namespace dopt
