// Convolution forward, backward-data and backward-filter as implicit GEMMs on fp32 MFMA.
// Replaces cudnnConvolutionForward / BackwardData / BackwardFilter as called at
// cuda/source/dopt/cuda/nnet/cudnn7.d:154, :199, :244.  The reference configures cuDNN with
// CUDNN_CONVOLUTION (cudnn7.d:87), i.e. a TRUE convolution: the filter is flipped,
//     y[n,k,p,q] = sum_{c,r,s} x[n,c,p*sy-ph+r, q*sx-pw+s] * w[k,c,R-1-r,S-1-s]
// (pinned by the known-answer test at core/source/dopt/core/ops/nnet.d:270-293).  Writing
// r' = R-1-r, s' = S-1-s the filter is read in plain memory order and the flip moves onto the
// input offset: x[n,c,p*sy-ph+(R-1-r'), q*sx-pw+(S-1-s')].
//
// Forward and backward-data share one "gather" kernel:
//     out[n,m,oh,ow] = sum_{tap,ci} Wp[tap,ci][m] * in[n,ci,ih(oh,tap),iw(ow,tap)]
// GEMM view: M = output channels of the op, columns = output pixels (n,oh,ow), reduction =
// (tap, ci) with ci padded to a multiple of 16 so that a 16-deep slab has ONE tap: the input
// offset and the bounds mask are then uniform over the slab, and a lane's loads for successive
// channels are one add apart.  Wp is the filter re-packed once per call into [tap*ci][m]
// (m contiguous), so the A tile goes global -> LDS with 128-bit accesses; the pack costs two
// passes over the filter, < 2 % of the layer's MFMA time for every VGG layer.
//
// Backward-filter is a GEMM with M = K (output channels), columns = (c,r',s') in filter memory
// order, reduction = output pixels (n,p,q); both operands are gathered with lanes along the
// pixel index (contiguous in memory).
//
// Layers with few output tiles (small spatial extent, or the short-and-wide filter gradients)
// split the reduction over blockIdx.y; partial tiles go to the workspace and are summed in a
// fixed order by a second kernel -- no float atomics, so results are reproducible.
#include "common.h"
#include "mfma_core.h"

namespace {

using namespace dopt;

constexpr int BK = 16;

struct GatherConv {
    const float *in;   // gathered operand [N, Cin, IH, IW]
    const float *wp;   // packed filter [taps * CinPad][Mp]
    float *out;        // [N, Mout, OH, OW], or `splits` partial copies of it
    int N, Cin, IH, IW, Mout, OH, OW, R, S;
    int padH, padW, strideH, strideW;
    int CinPad, Mp, ncols;
    int mtiles, ntiles, slabs_total, slabs_per_split;
    size_t out_elems;
};

template <int BM, bool kBwd>
__global__ __launch_bounds__(kGemmThreads, 2) void conv_gather_k(GatherConv p)
{
    constexpr int BN = BM == 128 ? 128 : 256, WN = BM == 128 ? 2 : 4;
    constexpr int LDA = BM + 4, LDB = BN + 4;
    constexpr int NA = BM * BK / 4 / kGemmThreads;  // float4 loads of A per thread
    constexpr int RSTEP = kGemmThreads / BN;        // reduction rows covered by one pass of B loads
    constexpr int NB = BK / RSTEP;                  // scalar loads of B per thread
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    unsigned L;
    if (!xcd_remap(blockIdx.x, (unsigned)(p.mtiles * p.ntiles), &L)) return;
    const int mt = (int)(L % (unsigned)p.mtiles), nt = (int)(L / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int split = blockIdx.y;
    const int slab_begin = split * p.slabs_per_split;
    const int slab_end = min(slab_begin + p.slabs_per_split, p.slabs_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / WN, wn = w % WN;

    // the output pixel this thread gathers for
    const int bcol = tid % BN, brow0 = tid / BN;
    const int pix = n0 + bcol;
    const bool pix_ok = pix < p.ncols;
    const int OHW = p.OH * p.OW;
    int n_img = 0, oh = 0, ow = 0;
    if (pix_ok) {
        n_img = pix / OHW;
        int pq = pix - n_img * OHW;
        oh = pq / p.OW;
        ow = pq - oh * p.OW;
    }
    const int chan_stride = p.IH * p.IW;
    const float *in_img = p.in + (size_t)n_img * p.Cin * chan_stride;

    float4 areg[NA];
    float breg[NB];

    auto load = [&](int slab) {
        const int kk0 = slab * BK;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int f = tid + kGemmThreads * i;
            const int row = f / (BM / 4), gm = m0 + (f % (BM / 4)) * 4;
            areg[i] = gm < p.Mp ? *(const float4 *)(p.wp + (size_t)(kk0 + row) * p.Mp + gm)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        const int tap = kk0 / p.CinPad, ci0 = kk0 - tap * p.CinPad;
        const int tr = tap / p.S, ts = tap - tr * p.S;
        int ih, iw;
        bool ok = pix_ok;
        if (!kBwd) {
            ih = oh * p.strideH - p.padH + (p.R - 1 - tr);
            iw = ow * p.strideW - p.padW + (p.S - 1 - ts);
        } else {
            // out = dx[.., h, w]; in = dy[.., ph, qw] with h = ph*stride - pad + r, r = R-1-tr
            const int nh = oh + p.padH - (p.R - 1 - tr), nw = ow + p.padW - (p.S - 1 - ts);
            ih = nh / p.strideH;
            iw = nw / p.strideW;
            ok = ok && nh >= 0 && nw >= 0 && ih * p.strideH == nh && iw * p.strideW == nw;
        }
        ok = ok && (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
        const float *src = in_img + ih * p.IW + iw;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int ci = ci0 + brow0 + RSTEP * i;
            breg[i] = (ok && ci < p.Cin) ? src[(size_t)ci * chan_stride] : 0.0f;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int f = tid + kGemmThreads * i;
            *(float4 *)&As[buf][(f / (BM / 4)) * LDA + (f % (BM / 4)) * 4] = areg[i];
        }
#pragma unroll
        for (int i = 0; i < NB; i++) Bs[buf][(brow0 + RSTEP * i) * LDB + bcol] = breg[i];
    };

    v16f acc[2][2];
    zero_acc(acc);
    load(slab_begin);
    store(0);
    __syncthreads();
    int cur = 0;
    for (int slab = slab_begin; slab < slab_end; ++slab) {
        const bool more = slab + 1 < slab_end;
        if (more) load(slab + 1);
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);
        if (more) store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    float *outp = p.out + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= p.ncols) continue;
        const int n2 = col / OHW, pq2 = col - n2 * OHW;
        float *base = outp + (size_t)n2 * p.Mout * OHW + pq2;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * 64 + i * 32 + acc_row(v, lane);
                if (m < p.Mout) base[(size_t)m * OHW] = acc[i][j][v];
            }
    }
}

struct FilterGrad {
    const float *dy;  // [N, K, P, Q]
    const float *x;   // [N, C, H, W]
    float *out;       // [K, C*R*S] or `splits` partial copies
    int N, C, H, W, K, P, Q, R, S;
    int padH, padW, strideH, strideW;
    int ncols;        // C*R*S
    int npix;         // N*P*Q
    int mtiles, ntiles, slabs_total, slabs_per_split;
    size_t out_elems;
};

template <int BM>
__global__ __launch_bounds__(kGemmThreads, 2) void conv_wgrad_k(FilterGrad p)
{
    constexpr int BN = BM == 128 ? 128 : 256, WN = BM == 128 ? 2 : 4;
    constexpr int LDA = BM + 4, LDB = BN + 4;
    constexpr int NA = BM / 16, NB = BN / 16;  // scalar loads per thread: lanes run along the pixel index
    __shared__ float As[2][BK * LDA];
    __shared__ float Bs[2][BK * LDB];

    unsigned L;
    if (!xcd_remap(blockIdx.x, (unsigned)(p.mtiles * p.ntiles), &L)) return;
    const int mt = (int)(L % (unsigned)p.mtiles), nt = (int)(L / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int split = blockIdx.y;
    const int slab_begin = split * p.slabs_per_split;
    const int slab_end = min(slab_begin + p.slabs_per_split, p.slabs_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / WN, wn = w % WN;
    const int kl = tid & 15, r0 = tid >> 4;  // reduction row inside the slab; first tile row/column
    const int PQ = p.P * p.Q, HW = p.H * p.W, taps = p.R * p.S;

    // per filter column (c, r', s') handled by this thread: channel offset and input displacement
    int coff[NB], dr[NB], ds[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        const int nn = n0 + r0 + 16 * i;
        if (nn < p.ncols) {
            const int c = nn / taps, tp = nn - c * taps;
            const int tr = tp / p.S, ts = tp - tr * p.S;
            coff[i] = c * HW;
            dr[i] = p.R - 1 - tr - p.padH;
            ds[i] = p.S - 1 - ts - p.padW;
        } else {
            coff[i] = 0;
            dr[i] = -(1 << 28);  // fails every bounds test
            ds[i] = 0;
        }
    }

    float areg[NA], breg[NB];
    auto load = [&](int slab) {
        const int kk = slab * BK + kl;
        const bool ok = kk < p.npix;
        int n = 0, ph = 0, qw = 0, pq = 0;
        if (ok) {
            n = kk / PQ;
            pq = kk - n * PQ;
            ph = pq / p.Q;
            qw = pq - ph * p.Q;
        }
        const float *ap = p.dy + (size_t)n * p.K * PQ + pq;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int m = m0 + r0 + 16 * i;
            areg[i] = (ok && m < p.K) ? ap[(size_t)m * PQ] : 0.0f;
        }
        const float *xp = p.x + (size_t)n * p.C * HW;
        const int ih0 = ph * p.strideH, iw0 = qw * p.strideW;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int ih = ih0 + dr[i], iw = iw0 + ds[i];
            const bool in = ok && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
            breg[i] = in ? xp[coff[i] + ih * p.W + iw] : 0.0f;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NA; i++) As[buf][kl * LDA + r0 + 16 * i] = areg[i];
#pragma unroll
        for (int i = 0; i < NB; i++) Bs[buf][kl * LDB + r0 + 16 * i] = breg[i];
    };

    v16f acc[2][2];
    zero_acc(acc);
    load(slab_begin);
    store(0);
    __syncthreads();
    int cur = 0;
    for (int slab = slab_begin; slab < slab_end; ++slab) {
        const bool more = slab + 1 < slab_end;
        if (more) load(slab + 1);
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);
        if (more) store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    float *outp = p.out + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= p.ncols) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * 64 + i * 32 + acc_row(v, lane);
                if (m < p.K) outp[(size_t)m * p.ncols + col] = acc[i][j][v];
            }
    }
}

// out[i] = sum_s partial[s][i], s ascending.
__global__ __launch_bounds__(256) void splitk_reduce_k(size_t n, int splits, const float *partial, float *out)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float acc = partial[i];
        for (int s = 1; s < splits; s++) acc += partial[(size_t)s * n + i];
        out[i] = acc;
    }
}

// Forward pack: w[K][C][taps] -> Wp[(tap*CinPad + c)][Mp] (m = k contiguous), through a 64x64 LDS tile.
__global__ __launch_bounds__(256) void pack_fwd_k(int K, int C, int taps, int CinPad, int Mp, const float *w,
                                                   float *wp)
{
    __shared__ float tile[64][65];
    const int CT = C * taps;
    const int m0 = blockIdx.x * 64, col0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int m = m0 + ty + 4 * k, cc = col0 + tx;
        tile[ty + 4 * k][tx] = (m < K && cc < CT) ? w[(size_t)m * CT + cc] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int cc = col0 + ty + 4 * k, m = m0 + tx;
        if (cc < CT && m < K) {
            const int c = cc / taps, t = cc - c * taps;
            wp[(size_t)(t * CinPad + c) * Mp + m] = tile[tx][ty + 4 * k];
        }
    }
}

// Backward-data pack: w[K][C][taps] -> Wp[(tap*KPad + k)][Mp] (m = c contiguous).
// Block (k, 64-channel chunk) stages w[k][c0 .. c0+64][*] (contiguous) in LDS.
__global__ __launch_bounds__(256) void pack_bwd_k(int K, int C, int taps, int KPad, int Mp, const float *w, float *wp)
{
    extern __shared__ float stage[];  // 64 * taps floats
    const int k = blockIdx.x, c0 = blockIdx.y * 64;
    const int nc = min(64, C - c0);
    const float *src = w + ((size_t)k * C + c0) * taps;
    for (int i = threadIdx.x; i < nc * taps; i += 256) stage[i] = src[i];
    __syncthreads();
    for (int i = threadIdx.x; i < nc * taps; i += 256) {
        const int t = i / nc, c = i - t * nc;
        wp[(size_t)(t * KPad + k) * Mp + c0 + c] = stage[c * taps + t];
    }
}

int round_up(int v, int to) { return (v + to - 1) / to * to; }

int pick_splits(int tiles, int slabs_total)
{
    int want = (2 * num_cus() + tiles - 1) / tiles;      // aim at two workgroups per CU
    int max_by_depth = slabs_total / 4 > 0 ? slabs_total / 4 : 1;  // keep >= 4 slabs per split
    int s = want < max_by_depth ? want : max_by_depth;
    if (s > 64) s = 64;
    return s < 1 ? 1 : s;
}

int check_desc(const dopt_hip_conv_desc *d, size_t *P, size_t *Q, const char *who)
{
    DOPT_REQUIRE(d != nullptr, "%s: descriptor is null", who);
    DOPT_REQUIRE(d->strideH > 0 && d->strideW > 0, "%s: stride must be positive", who);
    DOPT_REQUIRE(d->N && d->C && d->H && d->W && d->K && d->R && d->S, "%s: empty tensor", who);
    DOPT_REQUIRE(d->H + 2 * d->padH >= d->R && d->W + 2 * d->padW >= d->S, "%s: filter larger than padded input", who);
    DOPT_REQUIRE(d->R * d->S <= 64, "%s: filters above 64 taps are not supported", who);
    *P = (d->H + 2 * d->padH - d->R) / d->strideH + 1;  // core/ops/nnet.d:71-87
    *Q = (d->W + 2 * d->padW - d->S) / d->strideW + 1;
    const size_t lim = (size_t)1 << 30;
    DOPT_REQUIRE(d->N * d->C * d->H * d->W < lim && d->N * d->K * *P * *Q < lim && d->K * d->C * d->R * d->S < lim,
                 "%s: tensors above 2^30 elements are not supported", who);
    return DOPT_HIP_OK;
}

// Shared host driver of forward (kBwd = false) and backward-data (kBwd = true).
template <bool kBwd>
int run_gather(const dopt_hip_conv_desc *d, size_t P, size_t Q, const float *in, const float *w, float *out)
{
    GatherConv g{};
    const int taps = (int)(d->R * d->S);
    g.N = (int)d->N;
    g.R = (int)d->R;
    g.S = (int)d->S;
    g.padH = (int)d->padH;
    g.padW = (int)d->padW;
    g.strideH = (int)d->strideH;
    g.strideW = (int)d->strideW;
    if (!kBwd) {
        g.Cin = (int)d->C; g.IH = (int)d->H; g.IW = (int)d->W;
        g.Mout = (int)d->K; g.OH = (int)P; g.OW = (int)Q;
    } else {
        g.Cin = (int)d->K; g.IH = (int)P; g.IW = (int)Q;
        g.Mout = (int)d->C; g.OH = (int)d->H; g.OW = (int)d->W;
    }
    g.CinPad = round_up(g.Cin, BK);
    g.Mp = round_up(g.Mout, 4);
    g.ncols = g.N * g.OH * g.OW;
    g.slabs_total = taps * g.CinPad / BK;
    g.out_elems = (size_t)g.ncols * g.Mout;
    const bool big = g.Mout > 64;
    const int BM = big ? 128 : 64, BN = big ? 128 : 256;
    g.mtiles = (g.Mout + BM - 1) / BM;
    g.ntiles = (g.ncols + BN - 1) / BN;
    const int tiles = g.mtiles * g.ntiles;
    int splits = pick_splits(tiles, g.slabs_total);
    g.slabs_per_split = (g.slabs_total + splits - 1) / splits;
    splits = (g.slabs_total + g.slabs_per_split - 1) / g.slabs_per_split;  // no empty split

    const size_t wp_elems = (size_t)taps * g.CinPad * g.Mp;
    const size_t wp_bytes = (wp_elems * sizeof(float) + 255) / 256 * 256;
    const size_t part_bytes = splits > 1 ? (size_t)splits * g.out_elems * sizeof(float) : 0;
    char *ws = (char *)workspace(wp_bytes + part_bytes);
    if (!ws) return DOPT_HIP_ERR_OOM;
    float *wp = (float *)ws;
    float *partial = (float *)(ws + wp_bytes);

    // pack the filter
    if (g.CinPad != g.Cin || g.Mp != g.Mout) DOPT_HIP_CHECK(hipMemsetAsync(wp, 0, wp_elems * sizeof(float), stream()));
    const int K = (int)d->K, C = (int)d->C;
    if (!kBwd) {
        dim3 grid((unsigned)((K + 63) / 64), (unsigned)((C * taps + 63) / 64));
        hipLaunchKernelGGL(pack_fwd_k, grid, dim3(256), 0, stream(), K, C, taps, g.CinPad, g.Mp, w, wp);
    } else {
        dim3 grid((unsigned)K, (unsigned)((C + 63) / 64));
        hipLaunchKernelGGL(pack_bwd_k, grid, dim3(256), (size_t)64 * taps * sizeof(float), stream(), K, C, taps,
                           g.CinPad, g.Mp, w, wp);
    }
    DOPT_LAUNCH_CHECK();

    g.in = in;
    g.wp = wp;
    g.out = splits > 1 ? partial : out;
    dim3 grid(xcd_grid((unsigned)tiles), (unsigned)splits);
    if (big)
        hipLaunchKernelGGL((conv_gather_k<128, kBwd>), grid, dim3(kGemmThreads), 0, stream(), g);
    else
        hipLaunchKernelGGL((conv_gather_k<64, kBwd>), grid, dim3(kGemmThreads), 0, stream(), g);
    DOPT_LAUNCH_CHECK();
    if (splits > 1) {
        size_t blocks = ceil_div(g.out_elems, (size_t)256);
        size_t cap = (size_t)num_cus() * 8;
        hipLaunchKernelGGL(splitk_reduce_k, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0, stream(),
                           g.out_elems, splits, partial, out);
        DOPT_LAUNCH_CHECK();
    }
    return DOPT_HIP_OK;
}

}  // namespace

extern "C" {

int dopt_hip_conv_fwd(const dopt_hip_conv_desc *d, const float *x, const float *w, float *y)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_fwd")) return rc;
    DOPT_REQUIRE(x && w && y, "dopt_hip_conv_fwd: null argument");
    DOPT_ENSURE_INIT();
    return run_gather<false>(d, P, Q, x, w, y);
}

int dopt_hip_conv_bwd_data(const dopt_hip_conv_desc *d, const float *dy, const float *w, float *dx)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_data")) return rc;
    DOPT_REQUIRE(dy && w && dx, "dopt_hip_conv_bwd_data: null argument");
    DOPT_ENSURE_INIT();
    return run_gather<true>(d, P, Q, dy, w, dx);
}

int dopt_hip_conv_bwd_filter(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_filter")) return rc;
    DOPT_REQUIRE(dy && x && dw, "dopt_hip_conv_bwd_filter: null argument");
    DOPT_ENSURE_INIT();
    FilterGrad f{};
    f.dy = dy;
    f.x = x;
    f.N = (int)d->N; f.C = (int)d->C; f.H = (int)d->H; f.W = (int)d->W;
    f.K = (int)d->K; f.P = (int)P; f.Q = (int)Q; f.R = (int)d->R; f.S = (int)d->S;
    f.padH = (int)d->padH; f.padW = (int)d->padW; f.strideH = (int)d->strideH; f.strideW = (int)d->strideW;
    f.ncols = f.C * f.R * f.S;
    f.npix = f.N * f.P * f.Q;
    f.out_elems = (size_t)f.K * f.ncols;
    f.slabs_total = (f.npix + BK - 1) / BK;
    const bool big = f.K > 64;
    const int BM = big ? 128 : 64, BN = big ? 128 : 256;
    f.mtiles = (f.K + BM - 1) / BM;
    f.ntiles = (f.ncols + BN - 1) / BN;
    const int tiles = f.mtiles * f.ntiles;
    int splits = pick_splits(tiles, f.slabs_total);
    f.slabs_per_split = (f.slabs_total + splits - 1) / splits;
    splits = (f.slabs_total + f.slabs_per_split - 1) / f.slabs_per_split;
    float *partial = nullptr;
    if (splits > 1) {
        partial = (float *)workspace((size_t)splits * f.out_elems * sizeof(float));
        if (!partial) return DOPT_HIP_ERR_OOM;
    }
    f.out = splits > 1 ? partial : dw;
    dim3 grid(xcd_grid((unsigned)tiles), (unsigned)splits);
    if (big)
        hipLaunchKernelGGL((conv_wgrad_k<128>), grid, dim3(kGemmThreads), 0, stream(), f);
    else
        hipLaunchKernelGGL((conv_wgrad_k<64>), grid, dim3(kGemmThreads), 0, stream(), f);
    DOPT_LAUNCH_CHECK();
    if (splits > 1) {
        size_t blocks = ceil_div(f.out_elems, (size_t)256);
        size_t cap = (size_t)num_cus() * 8;
        hipLaunchKernelGGL(splitk_reduce_k, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0, stream(),
                           f.out_elems, splits, partial, dw);
        DOPT_LAUNCH_CHECK();
    }
    return DOPT_HIP_OK;
}

}  // extern "C"
