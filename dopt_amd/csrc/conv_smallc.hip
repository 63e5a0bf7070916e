// 3x3, pad 1, unit-stride convolutions whose input has at most three channels (the first layer of
// an image network): forward and filter gradient.  Replaces cudnnConvolutionForward /
// cudnnConvolutionBackwardFilter (cuda/source/dopt/cuda/nnet/cudnn7.d:133-159, :203-249) for that
// shape only; every other shape runs in conv.hip.
//
// With C * 9 <= 27 reduction steps the general kernels, which move 16 channels per step, would
// multiply mostly zeros.  Here the whole reduction (27 padded to 28) is 14 v_mfma_f32_32x32x2
// steps, the filter lives in registers, and both kernels are bound by the one large tensor they
// touch (y written once, dy read once).
//
// A block works on "sub-tiles" of 128 consecutive pixels of one image (RT = 128 / W whole rows).
// The input rows around them sit in LDS with a one-pixel zero border, xs[c][RT + 2][W + 2]; pixel
// px of the sub-tile reads its 3x3 window at xs[c][px / W + r][px % W + s].  Reduction index
// kk = c * 9 + r * 3 + s multiplies w[k][c][2 - r][2 - s]: the reference convolves with the flipped
// filter (core/source/dopt/core/ops/nnet.d:270-293).
#include "common.h"
#include "mfma_core.h"

namespace {

using namespace dopt;

constexpr int kThreads = 256;
constexpr int kPix = 128;          // pixels per sub-tile
constexpr int kSteps = 14;         // ceil(27 / 2) MFMA steps over the reduction
constexpr int kPatchMax = 3 * 10 * 130;  // largest xs: eight sub-tiles of W = 128 or W = 8 (10 x 130 or 130 x 10 per channel)

struct SmallC {
    const float *x, *w, *bias, *dy;
    float *y, *partial;
    int N, C, H, W, K;
    int RT, wshift;                // rows per sub-tile; log2(W)
    int tiles, tiles_per_image, tiles_per_block, blocks;
    int G, groups_per_image;       // forward: sub-tiles per block (one per wavefront)
};

// Zero-bordered input rows p0-1 .. p0+rows of image n into xs[c][rows + 2][W + 2].  Image rows are whole
// 16-byte quads (W is a power of two >= 8, x is 16-byte aligned), so a thread's unit is a quad and its
// coordinates are shifts and compares; U quads per thread are in flight before the first is used.
// Rows outside the image arrive as zeros (clamped address, value masked), the border columns are
// written separately.
template <int U>
__device__ __forceinline__ void load_patch(const SmallC &p, int n, int p0, int rows, int nthreads, float *xs)
{
    const int PW = p.W + 2, PR = rows + 2, qshift = p.wshift - 2, qmask = (1 << qshift) - 1;
    const int nrows = p.C * PR, total = nrows << qshift;
    for (int base = threadIdx.x; base < total; base += U * nthreads) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = min(base + u * nthreads, total - 1);
            const int r = i >> qshift, q = i & qmask;
            const int c = (r >= PR) + (r >= 2 * PR), row = p0 - 1 + (r - c * PR);
            v[u] = *(const float4 *)(p.x + ((size_t)(n * p.C + c) * p.H + min(max(row, 0), p.H - 1)) * p.W + 4 * q);
            if (row < 0 || row >= p.H) v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int i = base + u * nthreads;
            if (i < total) {
                float *d = xs + (i >> qshift) * PW + 1 + 4 * (i & qmask);
                d[0] = v[u].x; d[1] = v[u].y; d[2] = v[u].z; d[3] = v[u].w;
            }
        }
    }
    for (int r = threadIdx.x; r < nrows; r += nthreads) {
        xs[r * PW] = 0.0f;
        xs[r * PW + PW - 1] = 0.0f;
    }
}

// offset of reduction index kk inside xs (a patch of `rows` image rows), relative to a pixel's window corner
__device__ __forceinline__ int window_offset(const SmallC &p, int kk, int rows)
{
    const int c = kk / 9, r = (kk % 9) / 3, s = kk % 3;
    return c * (rows + 2) * (p.W + 2) + r * (p.W + 2) + s;
}

// y[n, k, p, q] (+ bias[k]).  A block takes G consecutive sub-tiles of one image (a wavefront each)
// and 32 output channels: for every channel the block's wavefronts write G * 512 contiguous bytes at
// about the same time.  (One sub-tile and all 64 channels per block computes the same thing but
// leaves 512-byte pieces 4 KB apart: 1.7 TB/s of writes instead of the copy rate.)
__global__ __launch_bounds__(512) void smallc_fwd_k(SmallC p)
{
    __shared__ float xs[kPatchMax];
    __shared__ float ws[32 * 27];   // this block's 32 filters as stored, [k][c][3][3]
    unsigned L;
    if (!xcd_remap(blockIdx.x, (unsigned)p.blocks, &L)) return;
    const int groups = p.tiles / p.G;                       // (image, group of sub-tiles) pairs
    const int kt = (int)L / groups, grp = (int)L % groups;
    const int n = grp / p.groups_per_image, p0 = (grp % p.groups_per_image) * p.G * p.RT;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, r32 = lane & 31;
    const int red = p.C * 9, k0 = kt * 32, krows = min(32, p.K - k0), nthreads = 64 * p.G;
    {   // at most 32 * 27 filter values: up to fourteen per thread of the smallest block, all in flight at once
        const int count = krows * red;
        float v[14];
#pragma unroll
        for (int u = 0; u < 14; u++) v[u] = p.w[(size_t)k0 * red + min((int)threadIdx.x + u * nthreads, count - 1)];
#pragma unroll
        for (int u = 0; u < 14; u++)
            if ((int)threadIdx.x + u * nthreads < count) ws[threadIdx.x + u * nthreads] = v[u];
    }
    load_patch<2>(p, n, p0, p.G * p.RT, nthreads, xs);
    // Pixels are the rows of the MFMA tile and output channels its columns, so a lane ends up with four consecutive
    // pixels of ONE channel in four consecutive accumulators: a 16-byte store (with channels as rows a lane held four
    // channels of one pixel, sixteen 4-byte stores per column; the store unit takes as long for the one as for the other).
    const float bv = p.bias ? p.bias[min(k0 + r32, p.K - 1)] : 0.0f;   // accumulators start at the bias of their channel
    __syncthreads();

    // the filter as MFMA B operands: lane (i, half) holds w for channel k0 + i, step kk = 2 t + half
    float aw[kSteps];
    int koff[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; t++) {
        const int kk = 2 * t + half;
        const bool live = kk < red;
        const int c = kk / 9, r = (kk % 9) / 3, s = kk % 3;
        koff[t] = window_offset(p, live ? kk : 0, p.G * p.RT);
        const float wv = ws[(min(r32, krows - 1) * p.C + (live ? c : 0)) * 9 + (2 - r) * 3 + (2 - s)];
        aw[t] = (live && r32 < krows) ? wv : 0.0f;
    }
    // Four 32-pixel columns of this wavefront's sub-tile, one after the other: the stores of a finished
    // column drain while the next one multiplies (with all four columns multiplied first and stored last,
    // every wavefront of the chip computed at the same time and then wrote at the same time).
    const size_t plane = (size_t)p.H * p.W;
    float *out = p.y + ((size_t)n * p.K + k0 + r32) * plane + (size_t)p0 * p.W + wave * kPix + 4 * half;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int px = wave * kPix + j * 32 + r32;
        const int poff = (px >> p.wshift) * (p.W + 2) + (px & (p.W - 1));
        v16f acc;
#pragma unroll
        for (int v = 0; v < 16; v++) acc[v] = bv;
#pragma unroll
        for (int t = 0; t < kSteps; t++)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[poff + koff[t]], aw[t], acc, 0, 0, 0);
        if (r32 < krows) {
#pragma unroll
            for (int g = 0; g < 4; g++)   // accumulators 4g .. 4g + 3: pixels 8g + 4 half .. + 3 of the column
                *(float4 *)(out + j * 32 + 8 * g) = make_float4(acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]);
        }
    }
}

// partial[block][k][j] = sum over the block's pixels of dy[n, k, pixel] * window(pixel)[j], j = c*9 + r*3 + s
__global__ __launch_bounds__(kThreads) void smallc_wgrad_k(SmallC p)
{
    constexpr int LD = kPix + 1;
    __shared__ float dys[64 * LD];   // [k][pixel]; reused for the cross-wavefront sum at the end
    __shared__ float xs[kPatchMax];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, r32 = lane & 31;
    const bool j_live = r32 < p.C * 9;
    const int joff = window_offset(p, j_live ? r32 : 0, p.RT);
    const size_t plane = (size_t)p.H * p.W;

    v16f acc[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[mt][v] = 0.0f;

    unsigned L;   // XCD-contiguous ranges of sub-tiles, as in the forward kernel
    const bool active = xcd_remap(blockIdx.x, (unsigned)p.blocks, &L);
    const int first = active ? (int)L * p.tiles_per_block : 0;
    const int last = active ? min(first + p.tiles_per_block, p.tiles) : 0;
    // dy of a sub-tile (64 rows of 128 consecutive floats, eight 16-byte loads per thread) and the input
    // patch under it (at most 288 quads, two per thread) are fetched one sub-tile ahead, so
    // that the loads are in flight while the current one multiplies
    constexpr int XQ = 2;   // at most 3 channels x 3 rows x 32 quads (W = 128) for 256 threads
    const int PW = p.W + 2, PR = p.RT + 2, qshift = p.wshift - 2, qmask = (1 << qshift) - 1;
    const int prows = p.C * PR, pquads = prows << qshift;
    float4 pre[8];
    float4 xq[XQ];
    auto fetch = [&](int tile) {
        const int n = tile / p.tiles_per_image, p0 = (tile % p.tiles_per_image) * p.RT;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int f = i * kThreads + threadIdx.x, k = f >> 5, q4 = f & 31;
            pre[i] = *(const float4 *)(p.dy + ((size_t)n * p.K + min(k, p.K - 1)) * plane + (size_t)p0 * p.W + q4 * 4);
        }
#pragma unroll
        for (int u = 0; u < XQ; u++) {   // the same quads, rows and masks as load_patch
            const int i = min((int)threadIdx.x + u * kThreads, pquads - 1);
            const int r = i >> qshift, q = i & qmask;
            const int c = (r >= PR) + (r >= 2 * PR), row = p0 - 1 + (r - c * PR);
            xq[u] = *(const float4 *)(p.x + ((size_t)(n * p.C + c) * p.H + min(max(row, 0), p.H - 1)) * p.W + 4 * q);
            if (row < 0 || row >= p.H) xq[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    // the border columns of xs stay zero for the whole kernel
    for (int r = threadIdx.x; r < prows; r += kThreads) {
        xs[r * PW] = 0.0f;
        xs[r * PW + PW - 1] = 0.0f;
    }
    if (first < last) fetch(first);
    for (int tile = first; tile < last; tile++) {
        __syncthreads();   // the previous sub-tile's readers are done
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int f = i * kThreads + threadIdx.x, k = f >> 5, q4 = f & 31;
            const bool row = k < p.K;
            float *d = dys + k * LD + q4 * 4;
            d[0] = row ? pre[i].x : 0.0f;
            d[1] = row ? pre[i].y : 0.0f;
            d[2] = row ? pre[i].z : 0.0f;
            d[3] = row ? pre[i].w : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < XQ; u++) {
            const int i = threadIdx.x + u * kThreads;
            if (i < pquads) {
                float *d = xs + (i >> qshift) * PW + 1 + 4 * (i & qmask);
                d[0] = xq[u].x; d[1] = xq[u].y; d[2] = xq[u].z; d[3] = xq[u].w;
            }
        }
        __syncthreads();
        if (tile + 1 < last) fetch(tile + 1);
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int px = wave * 32 + 2 * t + half;
            const float b = j_live ? xs[(px >> p.wshift) * (p.W + 2) + (px & (p.W - 1)) + joff] : 0.0f;
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(dys[r32 * LD + px], b, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(dys[(32 + r32) * LD + px], b, acc[1], 0, 0, 0);
        }
    }
    __syncthreads();
    float *red = dys;   // [wave][k][j]: 4 * 64 * 32 floats
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int v = 0; v < 16; v++) red[(wave * 64 + mt * 32 + acc_row(v, lane)) * 32 + r32] = acc[mt][v];
    __syncthreads();
    if (!active) return;
    float *out = p.partial + (size_t)L * 64 * 32;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int o = i * kThreads + threadIdx.x;
        out[o] = (red[o] + red[2048 + o]) + (red[4096 + o] + red[6144 + o]);
    }
}

// dw[k][c][2 - r][2 - s] = sum over blocks of partial[block][k][c*9 + r*3 + s].  One wavefront per
// output: lane l adds blocks l, l + 64, ... (independent loads), then the lanes are folded in a fixed order.
__global__ __launch_bounds__(kThreads) void smallc_wgrad_sum_k(int blocks, int K, int C, const float *partial, float *dw)
{
    const int o = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (o >= K * C * 9) return;
    const int k = o / (C * 9), j = o - k * C * 9, c = j / 9, r = (j % 9) / 3, s = j % 3;
    const float *src = partial + (size_t)k * 32 + j;
    float acc = 0.0f;
    for (int b = lane; b < blocks; b += 64) acc += src[(size_t)b * 2048];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) dw[((size_t)k * C + c) * 9 + (2 - r) * 3 + (2 - s)] = acc;
}

bool smallc_setup(const dopt_hip_conv_desc *d, SmallC *p)
{
    if (d->R != 3 || d->S != 3 || d->padH != 1 || d->padW != 1 || d->strideH != 1 || d->strideW != 1) return false;
    if (d->C < 1 || d->C > 3 || d->K < 1 || d->K > 64) return false;
    const size_t W = d->W;
    if (W < 8 || W > 128 || (W & (W - 1)) != 0) return false;
    const size_t RT = kPix / W;
    if (d->H % RT != 0 || d->N * d->K * d->H * d->W >= (1ull << 31)) return false;
    p->N = (int)d->N; p->C = (int)d->C; p->H = (int)d->H; p->W = (int)W; p->K = (int)d->K;
    p->RT = (int)RT;
    p->wshift = __builtin_ctz((unsigned)W);
    p->tiles_per_image = (int)(d->H / RT);
    p->tiles = p->N * p->tiles_per_image;
    return true;
}

}  // namespace

namespace dopt {

bool conv_smallc_takes(const dopt_hip_conv_desc *d)
{
    SmallC p{};
    return smallc_setup(d, &p);
}

int conv_smallc_fwd(const dopt_hip_conv_desc *d, const float *x, const float *w, const float *bias, float *y, bool *done)
{
    SmallC p{};
    *done = false;
    if (!smallc_setup(d, &p) || !aligned16(x) || !aligned16(y)) return DOPT_HIP_OK;   // 16-byte loads of x, stores of y
    p.x = x; p.w = w; p.bias = bias; p.y = y;
    p.G = 1;
    for (int g = 2; g <= 8; g++)
        if (p.tiles_per_image % g == 0) p.G = g;
    p.groups_per_image = p.tiles_per_image / p.G;
    p.blocks = (p.tiles / p.G) * ((p.K + 31) / 32);
    hipLaunchKernelGGL(smallc_fwd_k, dim3(xcd_grid((unsigned)p.blocks)), dim3(64 * p.G), 0, stream(), p);
    DOPT_LAUNCH_CHECK();
    *done = true;
    return DOPT_HIP_OK;
}

int conv_smallc_wgrad(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw, bool *done)
{
    SmallC p{};
    *done = false;
    if (!smallc_setup(d, &p) || !aligned16(dy) || !aligned16(x)) return DOPT_HIP_OK;
    const int want = num_cus();
    p.tiles_per_block = (p.tiles + want - 1) / want;
    const int blocks = (p.tiles + p.tiles_per_block - 1) / p.tiles_per_block;
    p.partial = (float *)workspace((size_t)blocks * 64 * 32 * sizeof(float));
    if (!p.partial) return DOPT_HIP_ERR_OOM;
    p.x = x; p.dy = dy; p.blocks = blocks;
    hipLaunchKernelGGL(smallc_wgrad_k, dim3(xcd_grid((unsigned)blocks)), dim3(kThreads), 0, stream(), p);
    DOPT_LAUNCH_CHECK();
    const int outs = p.K * p.C * 9;
    hipLaunchKernelGGL(smallc_wgrad_sum_k, dim3((unsigned)((outs + 3) / 4)), dim3(kThreads), 0, stream(),
                       blocks, p.K, p.C, p.partial, dw);
    DOPT_LAUNCH_CHECK();
    *done = true;
    return DOPT_HIP_OK;
}

}  // namespace dopt
