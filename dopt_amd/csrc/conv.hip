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
    int mtiles, ntiles, slabs_total, slabs_per_split, splits;
    size_t out_elems, in_bytes, wp_bytes;
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

    // 1-D grid over (split, tile), tile fastest: the blocks an XCD receives work on neighbouring
    // tiles of the same slice of the reduction, whatever the ratio of tiles to splits
    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    if (!xcd_remap(blockIdx.x, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int slab_begin = split * p.slabs_per_split;
    const int slab_end = min(slab_begin + p.slabs_per_split, p.slabs_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / WN, wn = w % WN;

    const __amdgpu_buffer_rsrc_t rin = make_rsrc(p.in, p.in_bytes);
    const __amdgpu_buffer_rsrc_t rwp = make_rsrc(p.wp, p.wp_bytes);

    // A: this thread's float4 slots of the [BK][BM] filter tile; byte offset relative to the slab's first row
    unsigned a_voff[NA];
    int a_lds[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) {
        const int f = tid + kGemmThreads * i;
        const int row = f / (BM / 4), gm = m0 + (f % (BM / 4)) * 4;
        a_voff[i] = gm < p.Mp ? (unsigned)(row * p.Mp + gm) * 4u : kOobOffset;
        a_lds[i] = row * LDA + (f % (BM / 4)) * 4;
    }

    // B: the output pixel this thread gathers for
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
    const int pix_base = (n_img * p.Cin + brow0) * chan_stride;  // element offset of (n, channel brow0, 0, 0)
    const int row_limit = p.Cin - brow0;                          // rows with ci0 + RSTEP*i >= row_limit are padding

    // running position in the (tap, channel) reduction, advanced slab by slab without divisions
    int kk0 = slab_begin * BK;
    int tap = kk0 / p.CinPad, ci0 = kk0 - tap * p.CinPad;
    int tr = tap / p.S, ts = tap - tr * p.S;

    float4 areg[NA];
    float breg[NB];

    auto load = [&]() {
        const unsigned a_soff = (unsigned)(kk0 * p.Mp) * 4u;
#pragma unroll
        for (int i = 0; i < NA; i++) areg[i] = buffer_load_f32x4(rwp, a_voff[i], a_soff);
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
        const unsigned b_voff = ok ? (unsigned)(pix_base + ih * p.IW + iw) * 4u : kOobOffset;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int ci = ci0 + RSTEP * i;  // wave-uniform
            const unsigned voff = (p.CinPad == p.Cin || ci < row_limit) ? b_voff : kOobOffset;
            breg[i] = buffer_load_f32(rin, voff, (unsigned)(ci * chan_stride) * 4u);
        }
        kk0 += BK;
        ci0 += BK;
        if (ci0 == p.CinPad) {
            ci0 = 0;
            if (++ts == p.S) {
                ts = 0;
                ++tr;
            }
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NA; i++) *(float4 *)&As[buf][a_lds[i]] = areg[i];
#pragma unroll
        for (int i = 0; i < NB; i++) Bs[buf][(brow0 + RSTEP * i) * LDB + bcol] = breg[i];
    };

    v16f acc[2][2];
    zero_acc(acc);
    load();
    store(0);
    __syncthreads();
    int cur = 0;
    // steady state: no branches inside, so loads, MFMAs and LDS stores of one iteration form one block
    for (int slab = slab_begin; slab < slab_end - 1; ++slab) {
        load();
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);
        store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);

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
    float *out;       // `splits` partial copies of [K][taps * Cp] (tap-major columns)
    int N, C, H, W, K, P, Q, R, S;
    int padH, padW, strideH, strideW;
    int Cp;           // C rounded up to 16: a 16-column group never straddles two taps
    int ncols;        // taps * Cp
    int npix;         // N*P*Q
    int mtiles, ntiles, slabs_total, slabs_per_split, splits;
    size_t out_elems, dy_bytes, x_bytes;
};

// Backward-filter.  GEMM columns are ordered tap-major, (r', s', c) with c padded to Cp, so that the
// 16-column groups a thread loads share one filter tap: the input displacement and the bounds test
// are then per group, not per element, and successive channels differ by a wave-uniform offset.
// TPT = number of column groups of a tile that may belong to different taps (BN / gcd(BN, Cp)).
// The partial tiles are summed over the splits and permuted back to [K][C][R][S] by wgrad_reduce_k.
template <int BM, int TPT>
__global__ __launch_bounds__(kGemmThreads, 2) void conv_wgrad_k(FilterGrad p)
{
    constexpr int BN = BM == 128 ? 128 : 256, WN = BM == 128 ? 2 : 4;
    constexpr int LDA = BM + 4, LDB = BN + 4;
    constexpr int NA = BM / 16, NB = BN / 16;  // scalar loads per thread: lanes run along the pixel index
    constexpr int GSZ = NB / TPT;              // loads per tap group
    __shared__ float As[2][BK * LDA];
    __shared__ float Bs[2][BK * LDB];

    // 1-D grid over (split, tile), tile fastest: the blocks an XCD receives work on neighbouring
    // tiles of the same slice of the reduction, whatever the ratio of tiles to splits
    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    if (!xcd_remap(blockIdx.x, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int slab_begin = split * p.slabs_per_split;
    const int slab_end = min(slab_begin + p.slabs_per_split, p.slabs_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / WN, wn = w % WN;
    const int kl = tid & 15, r0 = tid >> 4;  // reduction row inside the slab; first tile row/column
    const int PQ = p.P * p.Q, HW = p.H * p.W;

    const __amdgpu_buffer_rsrc_t rdy = make_rsrc(p.dy, p.dy_bytes);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x, p.x_bytes);

    // rows (output channels) at or past K are masked
    unsigned row_oob = 0;
#pragma unroll
    for (int i = 0; i < NA; i++)
        if (m0 + r0 + 16 * i >= p.K) row_oob |= 1u << i;
    const bool k_full = m0 + BM <= p.K;  // wave-uniform: every row of this tile exists

    // wave-uniform description of each tap group of this tile
    int g_dr[TPT], g_ds[TPT], g_disp[TPT], g_c0[TPT];
#pragma unroll
    for (int g = 0; g < TPT; g++) {
        const int nn = n0 + 16 * GSZ * g;
        if (nn < p.ncols) {
            const int tap = nn / p.Cp;
            const int tr = tap / p.S, ts = tap - tr * p.S;
            g_c0[g] = nn - tap * p.Cp;
            g_dr[g] = p.R - 1 - tr - p.padH;
            g_ds[g] = p.S - 1 - ts - p.padW;
        } else {
            g_c0[g] = 0;
            g_dr[g] = -(1 << 28);  // fails every bounds test
            g_ds[g] = 0;
        }
        g_disp[g] = g_dr[g] * p.W + g_ds[g];
    }
    const bool c_full = p.C == p.Cp;

    float areg[NA], breg[NB];
    auto load = [&](int slab) {
        const int kk = slab * BK + kl;
        const int oob_pix = (p.npix - 1 - kk);  // negative past the last pixel
        const int n = kk / PQ, pq = kk - n * PQ;
        const int ph = pq / p.Q, qw = pq - ph * p.Q;
        const unsigned a_raw = (unsigned)((n * p.K + m0 + r0) * PQ + pq) * 4u;
        const unsigned a_voff = oob_pix < 0 ? kOobOffset : a_raw;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            unsigned v = a_voff;
            if (!k_full) v = ((row_oob >> i) & 1u) ? kOobOffset : a_voff;
            areg[i] = buffer_load_f32(rdy, v, (unsigned)(16 * i * PQ) * 4u);
        }
        const int ih0 = ph * p.strideH, iw0 = qw * p.strideW;
        const int x_pix = (n * p.C + r0) * HW + ih0 * p.W + iw0;  // element offset of (n, channel r0, ih0, iw0)
#pragma unroll
        for (int g = 0; g < TPT; g++) {
            const int ih = ih0 + g_dr[g], iw = iw0 + g_ds[g];
            const int bad = ih | (p.H - 1 - ih) | iw | (p.W - 1 - iw) | oob_pix;  // sign bit: outside
            const unsigned g_voff = bad < 0 ? kOobOffset : (unsigned)(x_pix + g_disp[g]) * 4u;
#pragma unroll
            for (int ii = 0; ii < GSZ; ii++) {
                const int c_uni = g_c0[g] + 16 * ii;  // wave-uniform first channel of this load
                unsigned v = g_voff;
                if (!c_full) v = (c_uni + r0 < p.C) ? g_voff : kOobOffset;
                breg[g * GSZ + ii] = buffer_load_f32(rx, v, (unsigned)(c_uni * HW) * 4u);
            }
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
    for (int slab = slab_begin; slab < slab_end - 1; ++slab) {
        load(slab + 1);
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);
        store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * 64, wn * 64, acc, lane);

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

// dw[k][c][tap] = sum_s partial[s][k][tap*Cp + c], summed in a fixed order (reproducible).  Block
// (k, 16-channel chunk) reads tap rows coalesced, stages them in LDS and writes its 16*taps outputs
// contiguously.  Eight independent partial sums per element keep eight loads in flight: the split
// count reaches the hundreds for the wide early layers and a single dependent chain would be
// latency-bound.
__global__ __launch_bounds__(256) void wgrad_reduce_k(int K, int C, int Cp, int taps, int splits, size_t split_stride,
                                                       const float *partial, float *dw)
{
    extern __shared__ float stage[];  // [16][taps]
    const int k = blockIdx.x, c0 = blockIdx.y * 16;
    const int nc = min(16, C - c0);
    const float *src = partial + (size_t)k * taps * Cp + c0;
    for (int i = threadIdx.x; i < nc * taps; i += 256) {
        const int t = i / nc, c = i - t * nc;
        const float *q = src + (size_t)t * Cp + c;
        float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        int sp = 0;
        for (; sp + 8 <= splits; sp += 8) {
#pragma unroll
            for (int u = 0; u < 8; u++) a[u] += q[(size_t)(sp + u) * split_stride];
        }
        for (int u = 0; sp < splits; sp++, u++) a[u] += q[(size_t)sp * split_stride];
        stage[c * taps + t] = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
    }
    __syncthreads();
    float *dst = dw + ((size_t)k * C + c0) * taps;
    for (int i = threadIdx.x; i < nc * taps; i += 256) dst[i] = stage[i];
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

int pick_splits(int tiles, int slabs_total, int cap = 64)
{
    int want = (2 * num_cus() + tiles - 1) / tiles;      // aim at two workgroups per CU
    int max_by_depth = slabs_total / 4 > 0 ? slabs_total / 4 : 1;  // keep >= 4 slabs per split
    int s = want < max_by_depth ? want : max_by_depth;
    if (s > cap) s = cap;
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
    const size_t lim = (size_t)1 << 29;  // byte offsets of valid elements stay below 2^31
    DOPT_REQUIRE(d->N * d->C * d->H * d->W < lim && d->N * d->K * *P * *Q < lim && d->K * d->C * d->R * d->S < lim,
                 "%s: tensors of 2^29 elements or more are not supported", who);
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
    g.splits = splits;

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
    g.in_bytes = (size_t)g.N * g.Cin * g.IH * g.IW * sizeof(float);
    g.wp_bytes = wp_elems * sizeof(float);
    g.out = splits > 1 ? partial : out;
    dim3 grid(xcd_grid((unsigned)(tiles * splits)));
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
    const int taps = f.R * f.S;
    f.Cp = round_up(f.C, 16);
    f.ncols = taps * f.Cp;
    f.npix = f.N * f.P * f.Q;
    f.out_elems = (size_t)f.K * f.ncols;
    f.dy_bytes = (size_t)f.npix * f.K * sizeof(float);
    f.x_bytes = (size_t)f.N * f.C * f.H * f.W * sizeof(float);
    f.slabs_total = (f.npix + BK - 1) / BK;
    const bool big = f.K > 64;
    const int BM = big ? 128 : 64, BN = big ? 128 : 256;
    f.mtiles = (f.K + BM - 1) / BM;
    f.ntiles = (f.ncols + BN - 1) / BN;
    const int tiles = f.mtiles * f.ntiles;
    // filter gradients are short and wide (small output, long pixel reduction): allow deep splits
    int splits = pick_splits(tiles, f.slabs_total, 512);
    f.slabs_per_split = (f.slabs_total + splits - 1) / splits;
    splits = (f.slabs_total + f.slabs_per_split - 1) / f.slabs_per_split;
    f.splits = splits;
    float *partial = (float *)workspace((size_t)splits * f.out_elems * sizeof(float));
    if (!partial) return DOPT_HIP_ERR_OOM;
    f.out = partial;
    // column groups of one tile that can fall on different taps
    int gw = BN;
    while (f.Cp % gw != 0) gw /= 2;  // largest power-of-two divisor of Cp not above BN (>= 16)
    int tpt = BN / gw;
    if (tpt > 4) tpt = BN / 16;      // instantiated: 1, 2, 4 and one group per load
    dim3 grid(xcd_grid((unsigned)(tiles * splits)));
#define DOPT_WGRAD(BMV, TPTV) hipLaunchKernelGGL((conv_wgrad_k<BMV, TPTV>), grid, dim3(kGemmThreads), 0, stream(), f)
    if (big) {
        if (tpt == 1) DOPT_WGRAD(128, 1);
        else if (tpt == 2) DOPT_WGRAD(128, 2);
        else if (tpt == 4) DOPT_WGRAD(128, 4);
        else DOPT_WGRAD(128, 8);
    } else {
        if (tpt == 1) DOPT_WGRAD(64, 1);
        else if (tpt == 2) DOPT_WGRAD(64, 2);
        else if (tpt == 4) DOPT_WGRAD(64, 4);
        else DOPT_WGRAD(64, 16);
    }
#undef DOPT_WGRAD
    DOPT_LAUNCH_CHECK();
    dim3 rgrid((unsigned)f.K, (unsigned)((f.C + 15) / 16));
    hipLaunchKernelGGL(wgrad_reduce_k, rgrid, dim3(256), (size_t)16 * taps * sizeof(float), stream(), f.K, f.C, f.Cp,
                       taps, splits, f.out_elems, partial, dw);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

}  // extern "C"
