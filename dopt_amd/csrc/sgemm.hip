// `matmul`: row-major C[M,N] = A[M,K] * B[K,N] in fp32 (alpha = 1, beta = 0, no transposes).
// Replaces cublasSgemm_v2 at cuda/source/dopt/cuda/math.d:234-235.
//
// The reference funnels far more than dense layers through matmul: every scalar or bias
// broadcast is a product with a ones vector (core/source/dopt/core/ops/basic.d:370-381,
// core/source/dopt/core/ops/package.d:96-103) and rank-2 row / column sums are products with a
// ones vector too (core/source/dopt/core/ops/math.d:257-279).  Those degenerate shapes are
// HBM-bound and get their own kernels here; everything else runs on the fp32 MFMA tile engine.
#include "common.h"
#include "mfma_core.h"

namespace {

using namespace dopt;

constexpr int BK = 16;
constexpr int kGemmThreads = 256;

struct Gemm {
    const float *A, *B;
    float *C;  // or `splits` partial copies
    int M, N, K;
    int mtiles, ntiles, slabs_total, slabs_per_split, splits;
    size_t out_elems;
};

template <int BM, bool kVecB>
__global__ __launch_bounds__(kGemmThreads, 2) void sgemm_k(Gemm p)
{
    constexpr int BN = BM == 128 ? 128 : 256, WN = BM == 128 ? 2 : 4;
    constexpr int LDA = BM + 4, LDB = BN + 4;
    constexpr int NA = BM / 16;                     // A: lanes run along k (contiguous in memory)
    constexpr int NB4 = BN * BK / 4 / kGemmThreads; // B: float4 along n
    __shared__ float As[2][BK * LDA];
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
    const int kl = tid & 15, r0 = tid >> 4;

    float areg[NA];
    float4 breg[NB4];
    auto load = [&](int slab) {
        const int kk0 = slab * BK;
        const bool kok = kk0 + kl < p.K;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            const int m = m0 + r0 + 16 * i;
            areg[i] = (kok && m < p.M) ? p.A[(size_t)m * p.K + kk0 + kl] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < NB4; i++) {
            const int f = tid + kGemmThreads * i;
            const int row = f / (BN / 4), gn = n0 + (f % (BN / 4)) * 4;
            const int kk = kk0 + row;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (kk < p.K) {
                const float *src = p.B + (size_t)kk * p.N + gn;
                if (kVecB) {
                    if (gn < p.N) v = *(const float4 *)src;  // N % 4 == 0: a float4 never straddles the edge
                } else {
                    if (gn + 0 < p.N) v.x = src[0];
                    if (gn + 1 < p.N) v.y = src[1];
                    if (gn + 2 < p.N) v.z = src[2];
                    if (gn + 3 < p.N) v.w = src[3];
                }
            }
            breg[i] = v;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NA; i++) As[buf][kl * LDA + r0 + 16 * i] = areg[i];
#pragma unroll
        for (int i = 0; i < NB4; i++) {
            const int f = tid + kGemmThreads * i;
            *(float4 *)&Bs[buf][(f / (BN / 4)) * LDB + (f % (BN / 4)) * 4] = breg[i];
        }
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

    float *outp = p.C + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= p.N) continue;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * 64 + i * 32 + acc_row(v, lane);
                if (m < p.M) outp[(size_t)m * p.N + col] = acc[i][j][v];
            }
    }
}

__global__ __launch_bounds__(256) void splitk_reduce_k(size_t n, int splits, const float *partial, float *out)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float acc = partial[i];
        for (int s = 1; s < splits; s++) acc += partial[(size_t)s * n + i];
        out[i] = acc;
    }
}

// K == 1: C[m][n] = a[m] * b[n] -- the broadcast product.  One rounding per element, so a
// product with 1.0f reproduces the broadcast value exactly.
__global__ __launch_bounds__(256) void outer_k(size_t M, size_t N, const float *a, const float *b, float *c)
{
    const size_t total = M * N;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t m = i / N, n = i - m * N;
        c[i] = a[m] * b[n];
    }
}

// N == 1: C[m] = sum_k A[m][k] * b[k]; one wavefront per row, lanes along k.
__global__ __launch_bounds__(256) void gemv_rows_k(size_t M, size_t K, const float *A, const float *b, float *c)
{
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int lane = threadIdx.x & 63;
    const float *ar = A + row * K;
    float acc = 0.0f;
    for (size_t k = lane; k < K; k += 64) acc += ar[k] * b[k];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if (lane == 0) c[row] = acc;
}

// M == 1: C[n] = sum_k a[k] * B[k][n]; lanes along n, a block folds a slice of k; slices are then
// summed in a fixed order.
__global__ __launch_bounds__(256) void gemv_cols_k(size_t K, size_t N, size_t kslice, const float *a, const float *B,
                                                    float *partial)
{
    const size_t n = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    const size_t k0 = (size_t)blockIdx.y * kslice;
    const size_t k1 = k0 + kslice < K ? k0 + kslice : K;
    float acc = 0.0f;
    for (size_t k = k0; k < k1; k++) acc += a[k] * B[k * N + n];
    partial[(size_t)blockIdx.y * N + n] = acc;
}

unsigned flat_grid(size_t n)
{
    size_t blocks = ceil_div(n, (size_t)256);
    size_t cap = (size_t)num_cus() * 16;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace

extern "C" {

int dopt_hip_sgemm(size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    if (M * N == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(C != nullptr, "dopt_hip_sgemm: C is null");
    DOPT_ENSURE_INIT();
    if (K == 0) return dopt_hip_memset(C, 0, M * N * sizeof(float));  // beta = 0
    DOPT_REQUIRE(A && B, "dopt_hip_sgemm: null operand");
    DOPT_REQUIRE(M < ((size_t)1 << 30) && N < ((size_t)1 << 30) && K < ((size_t)1 << 30) &&
                     M * N < ((size_t)1 << 40),
                 "dopt_hip_sgemm: dimensions too large");

    if (K == 1) {
        hipLaunchKernelGGL(outer_k, dim3(flat_grid(M * N)), dim3(256), 0, stream(), M, N, A, B, C);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    if (N == 1) {
        hipLaunchKernelGGL(gemv_rows_k, dim3((unsigned)ceil_div(M, (size_t)4)), dim3(256), 0, stream(), M, K, A, B, C);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    if (M == 1) {
        size_t nblocks = ceil_div(N, (size_t)256);
        size_t slices = ceil_div((size_t)num_cus() * 2, nblocks);
        if (slices > ceil_div(K, (size_t)32)) slices = ceil_div(K, (size_t)32);
        if (slices > 64) slices = 64;
        if (slices < 1) slices = 1;
        size_t kslice = ceil_div(K, slices);
        slices = ceil_div(K, kslice);
        float *partial = C;
        if (slices > 1) {
            partial = (float *)workspace(slices * N * sizeof(float));
            if (!partial) return DOPT_HIP_ERR_OOM;
        }
        hipLaunchKernelGGL(gemv_cols_k, dim3((unsigned)nblocks, (unsigned)slices), dim3(256), 0, stream(), K, N, kslice,
                           A, B, partial);
        DOPT_LAUNCH_CHECK();
        if (slices > 1) {
            hipLaunchKernelGGL(splitk_reduce_k, dim3(flat_grid(N)), dim3(256), 0, stream(), N, (int)slices, partial, C);
            DOPT_LAUNCH_CHECK();
        }
        return DOPT_HIP_OK;
    }

    Gemm g{};
    g.A = A;
    g.B = B;
    g.M = (int)M;
    g.N = (int)N;
    g.K = (int)K;
    g.out_elems = M * N;
    g.slabs_total = (int)ceil_div(K, (size_t)BK);
    const bool big = M > 64;
    const int BM = big ? 128 : 64, BN = big ? 128 : 256;
    g.mtiles = (int)ceil_div(M, (size_t)BM);
    g.ntiles = (int)ceil_div(N, (size_t)BN);
    const int tiles = g.mtiles * g.ntiles;
    int want = (2 * num_cus() + tiles - 1) / tiles;
    int max_by_depth = g.slabs_total / 4 > 0 ? g.slabs_total / 4 : 1;
    int splits = want < max_by_depth ? want : max_by_depth;
    if (splits > 32) splits = 32;
    if (splits < 1) splits = 1;
    g.slabs_per_split = (g.slabs_total + splits - 1) / splits;
    splits = (g.slabs_total + g.slabs_per_split - 1) / g.slabs_per_split;
    g.splits = splits;
    float *partial = nullptr;
    if (splits > 1) {
        partial = (float *)workspace((size_t)splits * g.out_elems * sizeof(float));
        if (!partial) return DOPT_HIP_ERR_OOM;
    }
    g.C = splits > 1 ? partial : C;
    const bool vecB = (N % 4 == 0) && aligned16(B);
    dim3 grid(xcd_grid((unsigned)(tiles * splits)));
    if (big) {
        if (vecB) hipLaunchKernelGGL((sgemm_k<128, true>), grid, dim3(kGemmThreads), 0, stream(), g);
        else hipLaunchKernelGGL((sgemm_k<128, false>), grid, dim3(kGemmThreads), 0, stream(), g);
    } else {
        if (vecB) hipLaunchKernelGGL((sgemm_k<64, true>), grid, dim3(kGemmThreads), 0, stream(), g);
        else hipLaunchKernelGGL((sgemm_k<64, false>), grid, dim3(kGemmThreads), 0, stream(), g);
    }
    DOPT_LAUNCH_CHECK();
    if (splits > 1) {
        hipLaunchKernelGGL(splitk_reduce_k, dim3(flat_grid(g.out_elems)), dim3(256), 0, stream(), g.out_elems, splits,
                           partial, C);
        DOPT_LAUNCH_CHECK();
    }
    return DOPT_HIP_OK;
}

}  // extern "C"
