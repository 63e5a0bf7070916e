// `matmul`: row-major C[M,N] = A[M,K] * B[K,N] in fp32 (alpha = 1, beta = 0, no transposes).
// Replaces cublasSgemm_v2 at cuda/source/dopt/cuda/math.d:234-235.
//
// The reference funnels far more than dense layers through matmul: every scalar or bias
// broadcast is a product with a ones vector (core/source/dopt/core/ops/basic.d:370-381,
// core/source/dopt/core/ops/package.d:96-103) and rank-2 row / column sums are products with a
// ones vector too (core/source/dopt/core/ops/math.d:257-279).  Those degenerate shapes are
// HBM-bound and get their own kernels here; everything else runs on the fp32 MFMA tile engine.
#include <vector>

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
    int lda, ldb;  // row pitch of A and B as stored
    int mtiles, ntiles, slabs_total, slabs_per_split, splits;
    size_t out_elems;
    bool quads_a, quads_b;  // sgemm_rows_k: the k-contiguous operand can be read in 16-byte pieces
};

// An operand tile is BR rows (of M or of N) by BK reduction steps, staged k-major in LDS:
// Xs[k][r].  In memory the operand is either "k-contiguous" -- element (r, k) at X[r*ld + k],
// which is A as given or B transposed -- or "r-contiguous" -- element (r, k) at X[k*ld + r],
// which is B as given or A transposed.
//   k-contiguous: 16 lanes run along k, 16 row groups; the LDS store does the transposition.
//   r-contiguous: float4 along r, copied straight into the k-major tile.
template <int BR>
struct KContig {
    static constexpr int N = BR / 16;
    float reg[N];
    __device__ void load(const float *X, int ld, int r_base, int r_max, int kk0, int k_max, int tid)
    {
        const int kl = tid & 15, r0 = tid >> 4;
        const bool kok = kk0 + kl < k_max;
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int r = r_base + r0 + 16 * i;
            reg[i] = (kok && r < r_max) ? X[(size_t)r * ld + kk0 + kl] : 0.0f;
        }
    }
    __device__ void store(float *Xs, int LD, int tid) const
    {
        const int kl = tid & 15, r0 = tid >> 4;
#pragma unroll
        for (int i = 0; i < N; i++) Xs[kl * LD + r0 + 16 * i] = reg[i];
    }
};

template <int BR, bool kVec>
struct RContig {
    static constexpr int N = BR * BK / 4 / kGemmThreads;
    float4 reg[N];
    __device__ void load(const float *X, int ld, int r_base, int r_max, int kk0, int k_max, int tid)
    {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int f = tid + kGemmThreads * i;
            const int row = f / (BR / 4), gr = r_base + (f % (BR / 4)) * 4;
            const int kk = kk0 + row;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (kk < k_max) {
                const float *src = X + (size_t)kk * ld + gr;
                if (kVec) {
                    if (gr < r_max) v = *(const float4 *)src;  // r_max % 4 == 0: a float4 never straddles the edge
                } else {
                    if (gr + 0 < r_max) v.x = src[0];
                    if (gr + 1 < r_max) v.y = src[1];
                    if (gr + 2 < r_max) v.z = src[2];
                    if (gr + 3 < r_max) v.w = src[3];
                }
            }
            reg[i] = v;
        }
    }
    __device__ void store(float *Xs, int LD, int tid) const
    {
#pragma unroll
        for (int i = 0; i < N; i++) {
            const int f = tid + kGemmThreads * i;
            *(float4 *)&Xs[(f / (BR / 4)) * LD + (f % (BR / 4)) * 4] = reg[i];
        }
    }
};

template <bool kCond, class T, class F>
struct Pick {
    using type = T;
};
template <class T, class F>
struct Pick<false, T, F> {
    using type = F;
};

// C = op(A) * op(B).  kTA: A is stored [K][M]; kTB: B is stored [N][K].
template <int BM, bool kTA, bool kTB, bool kVec>
__global__ __launch_bounds__(kGemmThreads, 2) void sgemm_k(Gemm p)
{
    constexpr int BN = BM == 128 ? 128 : 256, WN = BM == 128 ? 2 : 4;
    constexpr int LDA = BM + 4, LDB = BN + 4;
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

    typename Pick<kTA, RContig<BM, kVec>, KContig<BM>>::type la;
    typename Pick<kTB, KContig<BN>, RContig<BN, kVec>>::type lb;
    auto load = [&](int slab) {
        la.load(p.A, p.lda, m0, p.M, slab * BK, p.K, tid);
        lb.load(p.B, p.ldb, n0, p.N, slab * BK, p.K, tid);
    };
    auto store = [&](int buf) {
        la.store(As[buf], LDA, tid);
        lb.store(Bs[buf], LDB, tid);
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

// The same product with row-major LDS tiles: Xs[r][k], 32 reduction steps per slab at a pitch of 36 floats, so that a
// lane's operands for eight steps are ONE 128-bit LDS read (lane half h takes steps 8g + 4h .. 8g + 4h + 3 on both
// operands - any pairing of steps works as long as A and B agree) instead of eight 32-bit reads: 16 LDS reads per
// 64 matrix instructions where the k-major tiles above need 128.  Every instruction a wavefront issues besides the
// matrix ones costs the matrix pipe about four cycles, which is what the large products lost.
//   k-contiguous operand: a thread copies 16-byte pieces, eight lanes per 128-byte row segment (whole cache lines);
//   r-contiguous operand: a thread gathers four reduction steps of one row with 4-byte loads (64 lanes = 256
//     contiguous bytes per load) and stores them as one quad - the transposition happens in registers.
// 128 x 128 tiles, four wavefronts of 64 x 64, two workgroups per CU.  It serves every product of more than 64 rows,
// whatever the operands' alignment and however they are transposed, so that one (M, N, K) always adds its terms in
// one order (a plan that reads a transposed operand in place gets the bits of the plan that copies it first).
constexpr int BK2 = 32, kPitch2 = BK2 + 4;

// Loads go through a buffer resource: an element outside the tile's rows or past the end of the reduction is fetched
// from kOobOffset, where the hardware range check returns zero, so the loop holds no branch and every load of a slab is
// in flight at once (guarded plain loads compile to one exec-masked region each, with waits in between).
template <bool kKContig, bool kQuads>
struct Stage2 {
    float4 q[4];        // the staged quads: 128 rows x 8 quads over 256 threads
    unsigned base[4];   // byte offset of quad i at reduction step 0, or kOobOffset when its row is outside the matrix
    int kq[4];          // first reduction step of quad i inside a slab
    unsigned step;      // bytes between consecutive reduction steps (r-contiguous: the row pitch)
    __device__ void init(int ld, int r_base, int r_max, int tid)
    {
        step = kKContig ? 4u : (unsigned)ld * 4u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int row;
            if (kKContig) {
                const int idx = tid + 256 * i;
                row = idx >> 3;
                kq[i] = 4 * (idx & 7);
            } else {
                row = tid & 127;
                kq[i] = 4 * ((tid >> 7) + 2 * i);
            }
            const int r = r_base + row;
            const unsigned at = kKContig ? ((unsigned)r * (unsigned)ld + (unsigned)kq[i]) * 4u
                                         : ((unsigned)kq[i] * (unsigned)ld + (unsigned)r) * 4u;
            base[i] = r < r_max ? at : kOobOffset;
        }
    }
    // kQuads: the rows of a k-contiguous operand are 16-byte addressable (pitch and the reduction's ends multiples of
    // 4, aligned base); otherwise its pieces are fetched element by element - same values, same order of the sums.
    // A slab wholly past the end of the reduction loads nothing (every offset out of range).
    __device__ void load(__amdgpu_buffer_rsrc_t rs, int k0, int k_max)
    {
        const unsigned soff = (unsigned)k0 * step;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int k = k0 + kq[i];
            if (kKContig && kQuads) {
                q[i] = buffer_load_f32x4(rs, k < k_max ? base[i] : kOobOffset, soff);
            } else {
                q[i].x = buffer_load_f32(rs, k + 0 < k_max ? base[i] : kOobOffset, soff);
                q[i].y = buffer_load_f32(rs, k + 1 < k_max ? base[i] + step : kOobOffset, soff);
                q[i].z = buffer_load_f32(rs, k + 2 < k_max ? base[i] + 2u * step : kOobOffset, soff);
                q[i].w = buffer_load_f32(rs, k + 3 < k_max ? base[i] + 3u * step : kOobOffset, soff);
            }
        }
    }
    __device__ void store(float *Xs, int tid) const
    {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = kKContig ? (tid + 256 * i) >> 3 : tid & 127;
            *(float4 *)&Xs[row * kPitch2 + kq[i]] = q[i];
        }
    }
};

template <bool kTA, bool kTB, bool kQA, bool kQB>
__global__ __launch_bounds__(kGemmThreads, 2) void sgemm_rows_k(Gemm p)
{
    constexpr int BM = 128, BN = 128;
    __shared__ __attribute__((aligned(16))) float As[2][BM * kPitch2];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN * kPitch2];

    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    if (!xcd_remap(blockIdx.x, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    // p.slabs_* count 16-step slabs (the other kernel's unit): two of them per slab here
    const int k_begin = split * p.slabs_per_split * BK;
    const int k_end = min(min(k_begin + p.slabs_per_split * BK, p.slabs_total * BK), p.K);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, l32 = lane & 31, kh = lane >> 5;
    const int wm = w >> 1, wn = w & 1;
    const int a_frag = (wm * 64 + l32) * kPitch2 + 4 * kh, b_frag = (wn * 64 + l32) * kPitch2 + 4 * kh;

    v16f acc[2][2];
    zero_acc(acc);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A, (size_t)p.M * p.K * sizeof(float));
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B, (size_t)p.K * p.N * sizeof(float));
    // Two register sets: while slab s is multiplied out of LDS, slab s + 1 waits in one set to be stored behind it and
    // slab s + 2 is on its way into the other, so a load has two slabs' worth of matrix work to arrive.  No branch
    // inside the loop: loads behind the last slab fall out of range and fetch nothing, their stores fill a buffer
    // nobody reads.
    Stage2<!kTA, kQA> la[2];   // A as given is k-contiguous
    Stage2<kTB, kQB> lb[2];    // B transposed is k-contiguous
#pragma unroll
    for (int u = 0; u < 2; u++) {
        la[u].init(p.lda, m0, p.M, tid);
        lb[u].init(p.ldb, n0, p.N, tid);
    }
    la[0].load(ra, k_begin, k_end);
    lb[0].load(rb, k_begin, k_end);
    la[1].load(ra, k_begin + BK2, k_end);
    lb[1].load(rb, k_begin + BK2, k_end);
    la[0].store(As[0], tid);
    lb[0].store(Bs[0], tid);
    __syncthreads();
    auto slab = [&](const float *as, const float *bs) {
#pragma unroll
        for (int g = 0; g < BK2 / 8; g++) {
            float4 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = *(const float4 *)(as + i * 32 * kPitch2 + 8 * g);
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = *(const float4 *)(bs + j * 32 * kPitch2 + 8 * g);
            // step by step over the four accumulators: consecutive matrix instructions never wait for each other
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const float av = e == 0 ? a[i].x : e == 1 ? a[i].y : e == 2 ? a[i].z : a[i].w;
                        const float bv = e == 0 ? b[j].x : e == 1 ? b[j].y : e == 2 ? b[j].z : b[j].w;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                    }
        }
    };
    // iteration pair: slab k0 from buffer 0 (set 1 holds k0 + 32, set 0 is refilled with k0 + 64), then slab k0 + 32
    // from buffer 1 (set 0 holds k0 + 64, set 1 is refilled with k0 + 96)
    for (int k0 = k_begin; k0 < k_end; k0 += 2 * BK2) {
        la[0].load(ra, k0 + 2 * BK2, k_end);
        lb[0].load(rb, k0 + 2 * BK2, k_end);
        slab(As[0] + a_frag, Bs[0] + b_frag);
        la[1].store(As[1], tid);
        lb[1].store(Bs[1], tid);
        __syncthreads();
        if (k0 + BK2 >= k_end) break;   // uniform
        la[1].load(ra, k0 + 3 * BK2, k_end);
        lb[1].load(rb, k0 + 3 * BK2, k_end);
        slab(As[1] + a_frag, Bs[1] + b_frag);
        la[0].store(As[0], tid);
        lb[0].store(Bs[0], tid);
        __syncthreads();
    }

    float *outp = p.C + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int col = n0 + wn * 64 + j * 32 + l32;
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

// Small outputs (a dense layer at batch 128: 128 x 512 values from a 512-deep reduction).  The tile
// engine above would run four blocks plus a reduction launch; here one block owns a 32 x 32 tile of
// C, its eight wavefronts each take an eighth of K straight from memory into MFMA operands (no LDS
// staging: nothing is reused inside a 32-wide tile), and the eight partial tiles are summed through
// LDS in wavefront order.  Per step of 8 reductions a lane holds four k values for its row of A and
// four for its column of B; v_mfma_f32_32x32x2 number e pairs element e of lanes 0-31 (k = 8q + e)
// with element e of lanes 32-63 (k = 8q + 4 + e) - any pairing works as long as A and B agree.
//
// X is "k-contiguous" when element (r, k) sits at X[r * ld + k] (A as given, B transposed), else
// "r-contiguous" at X[k * ld + r].
//
// Loads go through buffer resources (an element outside the matrix or past the end of the wavefront's share of K
// comes from kOobOffset and reads as zero: no branch) and kSmallDepth steps are in flight per wavefront: with one
// step of prefetch every step waited a full memory latency, eight of them in a row for a 512-deep reduction -
// most of such a kernel's duration.  The order of the sums is that of the steps, whatever is in flight.
constexpr int kSmallWaves = 8, kSmallDepth = 4;
constexpr int kGroupJobs = 8;   // jobs one grouped launch may hold (its descriptions travel as kernel arguments)

// The lane's four reductions kk .. kk + 3 of row / column r.  `base`: byte offset of (r, reduction 0), or kOobOffset
// when r lies outside the matrix; `pitch`: bytes between consecutive reductions of an r-contiguous operand.
template <bool kKContig, bool kVec>
__device__ __forceinline__ void small_load(__amdgpu_buffer_rsrc_t rs, unsigned base, unsigned pitch, int kk, int k_end,
                                           float (&v)[4])
{
    if (kKContig && kVec) {   // rows are whole quads: the end of the reduction never cuts one
        const float4 q = buffer_load_f32x4(rs, kk < k_end ? base + (unsigned)kk * 4u : kOobOffset, 0);
        v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    } else {
        const unsigned step = kKContig ? 4u : pitch;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = buffer_load_f32(rs, kk + e < k_end ? base + (unsigned)(kk + e) * step : kOobOffset, 0);
    }
}

// kVA / kVB: the rows of a k-contiguous A / B are 16-byte addressable (an r-contiguous operand has no use for the flag).
template <bool kTA, bool kTB, bool kVA, bool kVB>
__device__ __forceinline__ void sgemm_small_body(int M, int N, int K, int lda, int ldb, int kslice, const float *A,
                                                 const float *B, float *C, const float *colbias, int bias_shift,
                                                 const float *rowvec, int relu, const float *mask, int bx, int by,
                                                 float (*red)[32 * 33])
{
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, r = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: loop bounds stay scalar
    const int m0 = by * 32, n0 = bx * 32;
    const int row = m0 + r, col = n0 + r;
    const int k_begin = wave * kslice, k_end = min(K, k_begin + kslice);
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc(A, (size_t)M * K * sizeof(float)), rsb = make_rsrc(B, (size_t)K * N * sizeof(float));
    // A is k-contiguous as given, B when it is read transposed
    const unsigned abase = row < M ? (kTA ? (unsigned)row * 4u : (unsigned)row * (unsigned)lda * 4u) : kOobOffset;
    const unsigned bbase = col < N ? (kTB ? (unsigned)col * (unsigned)ldb * 4u : (unsigned)col * 4u) : kOobOffset;
    const unsigned apitch = (unsigned)lda * 4u, bpitch = (unsigned)ldb * 4u;

    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
    float a[kSmallDepth][4], b[kSmallDepth][4];
    const int nsteps = k_begin < k_end ? (k_end - k_begin + 7) / 8 : 0;
#pragma unroll
    for (int j = 0; j < kSmallDepth; j++) {   // steps past the end fetch nothing
        small_load<!kTA, kVA>(rsa, abase, apitch, k_begin + 8 * j + 4 * half, k_end, a[j]);
        small_load<kTB, kVB>(rsb, bbase, bpitch, k_begin + 8 * j + 4 * half, k_end, b[j]);
        __builtin_amdgcn_sched_barrier(0);   // in this order: the first step's operands are waited for first
    }
    // Whole rounds of kSmallDepth steps without a branch inside (a branch per step made the compiler wait for every
    // load in flight at the top of the loop), then the steps left over, whose operands are in their registers or on
    // their way already.
    const int whole = nsteps / kSmallDepth * kSmallDepth;
    for (int s = 0; s < whole; s += kSmallDepth) {
#pragma unroll
        for (int j = 0; j < kSmallDepth; j++) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j][e], b[j][e], acc, 0, 0, 0);
            const int kk = k_begin + 8 * (s + j + kSmallDepth) + 4 * half;   // this register set's next step
            small_load<!kTA, kVA>(rsa, abase, apitch, kk, k_end, a[j]);
            small_load<kTB, kVB>(rsb, bbase, bpitch, kk, k_end, b[j]);
            __builtin_amdgcn_sched_barrier(0);   // keep each refill behind its own step: sunk to the loop's end, all of them are waited for at once
        }
    }
#pragma unroll
    for (int j = 0; j < kSmallDepth - 1; j++)
        if (whole + j < nsteps) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j][e], b[j][e], acc, 0, 0, 0);
        }
#pragma unroll
    for (int v = 0; v < 16; v++) red[wave][acc_row(v, lane) * 33 + r] = acc[v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int idx = tid + i * 64 * kSmallWaves, rr = idx >> 5, cc = idx & 31;
        float sum = red[0][rr * 33 + cc];
#pragma unroll
        for (int w = 1; w < kSmallWaves; w++) sum += red[w][rr * 33 + cc];
        if (m0 + rr < M && n0 + cc < N) {
            if (colbias) {   // one value per group of 2^bias_shift columns, times the row's factor when there is one
                float add = colbias[(n0 + cc) >> bias_shift];
                if (rowvec) add = __fmul_rn(rowvec[m0 + rr], add);   // rounded on its own, as the separate product is
                sum += add;
            }
            if (relu) sum = sum < 0.0f ? 0.0f : sum;
            if (mask) sum = mask[(size_t)(m0 + rr) * N + n0 + cc] > 0.0f ? sum : 0.0f;   // reluGrad(product, ., mask)
            C[(size_t)(m0 + rr) * N + n0 + cc] = sum;
        }
    }
}

template <bool kTA, bool kTB, bool kVA, bool kVB>
__global__ __launch_bounds__(64 * kSmallWaves) void sgemm_small_k(int M, int N, int K, int lda, int ldb, int kslice,
                                                                   const float *A, const float *B, float *C,
                                                                   const float *colbias, int bias_shift,
                                                                   const float *rowvec, int relu, const float *mask)
{
    __shared__ float red[kSmallWaves][32 * 33];
    sgemm_small_body<kTA, kTB, kVA, kVB>(M, N, K, lda, ldb, kslice, A, B, C, colbias, bias_shift, rowvec, relu, mask,
                                         (int)blockIdx.x, (int)blockIdx.y, red);
}

// Short reductions over large outputs with both operands stored k-major (A as [K][M], B as [K][N]:
// the product x^T * dy of a filter gradient).  With K <= 128 a 128 x 128 output tile needs 128 KB of
// operands, which fit in LDS whole: every load of the block is issued before the first multiply, so
// the memory latency is paid once per tile instead of once per slab, and each operand byte enters
// the CU once per 128 x 128 outputs (a quarter of what 32 x 32 tiles fetch).  The reduction runs in
// four chunks of 32; a chunk is multiplied as soon as it is in LDS while the later ones are still
// in flight.  Eight wavefronts as 2 x 4, 64 x 32 outputs each.
constexpr int kPanelK = 128, kPanelTile = 128, kPanelThreads = 512, kPanelLd = kPanelTile + 4;
constexpr size_t kPanelLds = (size_t)2 * kPanelK * kPanelLd * sizeof(float);

// Element (k, r .. r + 3) of an operand stored [K][R] (R % 4 == 0, 16-byte aligned), zero outside.
__device__ __forceinline__ float4 panel_load(const float *X, int ld, int k, int K, int r, int R)
{
    return (k < K && r < R) ? *(const float4 *)(X + (size_t)k * ld + r) : make_float4(0.f, 0.f, 0.f, 0.f);
}

// kFold: the product is the filter gradient of a 3x3, pad-1 convolution over 2x2 images written as a
// dense product -- row 4c + (input pixel), column 4k + (output pixel) -- and the kernel stores the
// nine tap sums of every (k, c) pair to C[k][c][3][3] instead of the 4 x 4 block itself: tap (a, b)
// collects the pixel pairs with 1 - iy + oy == a and 1 - ix + ox == b.
template <bool kFold>
__device__ __forceinline__ void sgemm_panel_body(int M, int N, int K, int mtiles, int ntiles, const float *A, const float *B,
                                                 float *C, unsigned bid)
{
    extern __shared__ __attribute__((aligned(16))) float panel_lds[];
    float *As = panel_lds, *Bs = panel_lds + kPanelK * kPanelLd;
    unsigned L;
    if (!xcd_remap(bid, (unsigned)(mtiles * ntiles), &L)) return;
    const int m0 = (int)(L % (unsigned)mtiles) * kPanelTile, n0 = (int)(L / (unsigned)mtiles) * kPanelTile;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, wm = w >> 2, wn = w & 3;

    // chunk c = reduction steps [32c, 32c + 32): 1024 float4 per operand, two per thread
    float4 ra[4][2], rb[4][2];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int f = tid + kPanelThreads * i, k = 32 * c + (f >> 5), r = (f & 31) * 4;
            ra[c][i] = panel_load(A, M, k, K, m0 + r, M);
            rb[c][i] = panel_load(B, N, k, K, n0 + r, N);
        }
    v16f acc[2][1];
    zero_acc(acc);
#pragma unroll
    for (int c = 0; c < 4; c++) {
        if (32 * c < K) {   // uniform
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int f = tid + kPanelThreads * i, o = (32 * c + (f >> 5)) * kPanelLd + (f & 31) * 4;
                *(float4 *)&As[o] = ra[c][i];
                *(float4 *)&Bs[o] = rb[c][i];
            }
            __syncthreads();
            mma_slab<32, kPanelLd, kPanelLd>(As + 32 * c * kPanelLd, Bs + 32 * c * kPanelLd, wm * 64, wn * 32, acc, lane);
        }
    }
    if constexpr (!kFold) {
        const int col = n0 + wn * 32 + (lane & 31);
        if (col < N) {
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + wm * 64 + i * 32 + acc_row(v, lane);
                    if (m < M) C[(size_t)m * N + col] = acc[i][0][v];
                }
        }
    } else {
        // the tile goes back through LDS (the operands are spent) so that one thread sees the 4 x 4
        // block of a (c, k) pair; threads run along c, which is contiguous in the filter gradient
        __syncthreads();
        float *tile = panel_lds;   // [128][kPanelLd]
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                tile[(wm * 64 + i * 32 + acc_row(v, lane)) * kPanelLd + wn * 32 + (lane & 31)] = acc[i][0][v];
        __syncthreads();
        const int Cin = M / 4, Kout = N / 4;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int pair = tid + kPanelThreads * j, cl = pair & 31, kl = pair >> 5;
            const int c = m0 / 4 + cl, k = n0 / 4 + kl;
            if (c < Cin && k < Kout) {
                float q[4][4];   // [input pixel iy*2+ix][output pixel oy*2+ox]
#pragma unroll
                for (int pin = 0; pin < 4; pin++) {
                    const float4 v = *(const float4 *)&tile[(cl * 4 + pin) * kPanelLd + kl * 4];
                    q[pin][0] = v.x; q[pin][1] = v.y; q[pin][2] = v.z; q[pin][3] = v.w;
                }
                float *out = C + ((size_t)k * Cin + c) * 9;
#pragma unroll
                for (int a = 0; a < 3; a++)
#pragma unroll
                    for (int b = 0; b < 3; b++) {
                        float sum = 0.0f;
#pragma unroll
                        for (int iy = 0; iy < 2; iy++)
#pragma unroll
                            for (int ix = 0; ix < 2; ix++) {
                                const int oy = a - 1 + iy, ox = b - 1 + ix;
                                if (oy >= 0 && oy < 2 && ox >= 0 && ox < 2) sum += q[iy * 2 + ix][oy * 2 + ox];
                            }
                        out[a * 3 + b] = sum;
                    }
            }
        }
    }
}

template <bool kFold>
__global__ __launch_bounds__(kPanelThreads) void sgemm_panel_k(int M, int N, int K, int mtiles, int ntiles, const float *A,
                                                                const float *B, float *C)
{
    sgemm_panel_body<kFold>(M, N, K, mtiles, ntiles, A, B, C, blockIdx.x);
}

// Several such products in one launch (the filter gradients of consecutive 2x2-image layers wait for nothing but their
// own dy): job j owns the blocks from first[j] on, a multiple of 8 each, so a block's place among the XCDs is what it
// would be in a launch of its own.
struct PanelJob {
    int M, N, K, mtiles, ntiles;
    unsigned first;
    const float *A, *B;
    float *C;
};
struct PanelGroup {
    PanelJob j[kGroupJobs];
    int n;
};

template <bool kFold>
__global__ __launch_bounds__(kPanelThreads) void sgemm_panel_group_k(PanelGroup g)
{
    int j = 0;
    while (j + 1 < g.n && blockIdx.x >= g.j[j + 1].first) j++;
    const PanelJob &q = g.j[j];
    sgemm_panel_body<kFold>(q.M, q.N, q.K, q.mtiles, q.ntiles, q.A, q.B, q.C, blockIdx.x - q.first);
}

__global__ __launch_bounds__(256) void splitk_reduce_k(size_t n, int splits, const float *partial, float *out)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        // four loads in flight per round (indices clamped, surplus values dropped); adds in split order
        float acc = 0.f;
        const int last = splits - 1;
        for (int s = 0; s < splits; s += 4) {
            const float v0 = partial[(size_t)s * n + i], v1 = partial[(size_t)min(s + 1, last) * n + i];
            const float v2 = partial[(size_t)min(s + 2, last) * n + i], v3 = partial[(size_t)min(s + 3, last) * n + i];
            acc = (((acc + v0) + (s + 1 <= last ? v1 : 0.f)) + (s + 2 <= last ? v2 : 0.f)) + (s + 3 <= last ? v3 : 0.f);
        }
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

// The same for a short reduction (K <= 256) in one launch: a block takes 64 columns, its four
// groups of 64 threads take every fourth k, sixteen loads in flight per thread (clamped, not
// branched), and the four sums are added in group order through LDS.
// (`on`: false for the threads of a larger block that only keep the barrier company)
__device__ __forceinline__ void gemv_cols_short_body(int K, int N, const float *a, const float *B, float *c, int bx, bool on,
                                                     float (*part)[64])
{
    const int col = threadIdx.x & 63, kl = (threadIdx.x >> 6) & 3;
    const int n = min(bx * 64 + col, N - 1);
    float acc = 0.0f;
    if (on) {
        for (int k0 = kl; k0 < K; k0 += 64) {
            float av[16], bv[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const int k = min(k0 + 4 * u, K - 1);
                av[u] = a[k];
                bv[u] = B[(size_t)k * N + n];
            }
#pragma unroll
            for (int u = 0; u < 16; u++)
                if (k0 + 4 * u < K) acc += av[u] * bv[u];
        }
        part[kl][col] = acc;
    }
    __syncthreads();
    if (on && kl == 0 && bx * 64 + col < N) c[n] = ((part[0][col] + part[1][col]) + part[2][col]) + part[3][col];
}

__global__ __launch_bounds__(256) void gemv_cols_short_k(int K, int N, const float *a, const float *B, float *c)
{
    __shared__ float part[4][64];
    gemv_cols_short_body(K, N, a, B, c, (int)blockIdx.x, true, part);
}

// Several independent small products in ONE launch: the weight and bias gradients of a dense head are six kernels of a
// few microseconds each that wait for nothing but the gradient in front of them, and a kernel boundary costs as much as
// one of them runs.  A block finds its job by its index; each job runs the body of the kernel it would have run alone
// (32 x 32-tile products of one template instance, and column sums of short reductions), so every value is what the
// separate launches give.
struct SmallJob {
    int M, N, K, lda, ldb, kslice, nx, first;   // nx: tiles per row of tiles; first: the job's first block
    const float *A, *B;
    float *C;
};
struct GemvJob {
    int K, N, first, pad;
    const float *a, *B;
    float *c;
};
struct SmallGroup {
    SmallJob s[kGroupJobs];
    GemvJob v[kGroupJobs];
    int ns, nv;
};

template <bool kTA, bool kTB, bool kVA, bool kVB>
__global__ __launch_bounds__(64 * kSmallWaves) void sgemm_small_group_k(SmallGroup g)
{
    __shared__ float red[kSmallWaves][32 * 33];
    __shared__ float part[4][64];
    const int b = (int)blockIdx.x;   // uniform: the scans below stay scalar
    if (g.nv > 0 && b >= g.v[0].first) {
        int j = 0;
        while (j + 1 < g.nv && b >= g.v[j + 1].first) j++;
        const GemvJob &q = g.v[j];
        gemv_cols_short_body(q.K, q.N, q.a, q.B, q.c, b - q.first, threadIdx.x < 256, part);
        return;
    }
    int j = 0;
    while (j + 1 < g.ns && b >= g.s[j + 1].first) j++;
    const SmallJob &q = g.s[j];
    const int local = b - q.first;
    sgemm_small_body<kTA, kTB, kVA, kVB>(q.M, q.N, q.K, q.lda, q.ldb, q.kslice, q.A, q.B, q.C, nullptr, 0, nullptr, 0, nullptr,
                                         local % q.nx, local / q.nx, red);
}

// c[m][n] = relu?(c[m][n] + u[m] * v[n]): the epilogue of dopt_hip_sgemm_rank1 as a pass of its own, for the
// shapes whose product kernel has none.  Each step rounds on its own, like the separate operations.
__global__ __launch_bounds__(256) void rank1_epilogue_k(size_t M, size_t N, const float *u, const float *v, int relu, float *c)
{
    const size_t total = M * N;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t m = i / N, n = i - m * N;
        float x = c[i];
        if (v) x += __fmul_rn(u[m], v[n]);
        if (relu) x = x < 0.0f ? 0.0f : x;
        c[i] = x;
    }
}

unsigned flat_grid(size_t n)
{
    size_t blocks = ceil_div(n, (size_t)256);
    size_t cap = (size_t)num_cus() * 16;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

// The LDS-resident kernel wins where its 128 x 128 tiles give every CU one or two blocks and the
// operands take 128-bit loads (2048 x 2048 x 128: 17 us against 22 us for the 32 x 32 tiles); with
// fewer tiles CUs idle, with more the tile engine's two resident blocks per CU overlap better.
bool panel_shape(size_t M, size_t N, size_t K)
{
    const size_t tiles = ceil_div(M, (size_t)kPanelTile) * ceil_div(N, (size_t)kPanelTile);
    return K >= 1 && K <= (size_t)kPanelK && tiles >= (size_t)num_cus() && tiles <= (size_t)2 * num_cus() && M % 4 == 0 &&
           N % 4 == 0;
}

bool panel_takes(size_t M, size_t N, size_t K, const float *A, const float *B)
{
    return panel_shape(M, N, K) && aligned16(A) && aligned16(B);
}

int panel_launch(bool fold, size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    static bool raised = false;
    if (!raised) {   // above 64 KB of dynamic LDS a kernel has to be told once
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)sgemm_panel_k<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kPanelLds));
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)sgemm_panel_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kPanelLds));
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)sgemm_panel_group_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kPanelLds));
        raised = true;
    }
    if (M == 0) return DOPT_HIP_OK;   // called for the attributes only
    const int mt = (int)ceil_div(M, (size_t)kPanelTile), nt = (int)ceil_div(N, (size_t)kPanelTile);
    const dim3 grid(xcd_grid((unsigned)(mt * nt))), block(kPanelThreads);
    if (fold) hipLaunchKernelGGL(sgemm_panel_k<true>, grid, block, kPanelLds, stream(), (int)M, (int)N, (int)K, mt, nt, A, B, C);
    else hipLaunchKernelGGL(sgemm_panel_k<false>, grid, block, kPanelLds, stream(), (int)M, (int)N, (int)K, mt, nt, A, B, C);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// `n` folded filter-gradient products (all of them shapes panel_takes accepts) as one launch.
int panel_fold_group_launch(int n, const size_t *M, const size_t *N, const size_t *K, const float *const *A,
                            const float *const *B, float *const *C)
{
    if (int rc = panel_launch(true, 0, 0, 0, nullptr, nullptr, nullptr)) return rc;
    PanelGroup g{};
    unsigned blocks = 0;
    for (int i = 0; i < n; i++) {
        PanelJob &q = g.j[i];
        q.M = (int)M[i]; q.N = (int)N[i]; q.K = (int)K[i];
        q.mtiles = (int)ceil_div(M[i], (size_t)kPanelTile);
        q.ntiles = (int)ceil_div(N[i], (size_t)kPanelTile);
        q.first = blocks;
        q.A = A[i]; q.B = B[i]; q.C = C[i];
        blocks += xcd_grid((unsigned)(q.mtiles * q.ntiles));
    }
    g.n = n;
    hipLaunchKernelGGL(sgemm_panel_group_k<true>, dim3(blocks), dim3(kPanelThreads), kPanelLds, stream(), g);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

}  // namespace

namespace dopt {

// C[M,N] = op(A) * op(B) with op(X) = X or its transpose: transA means A is stored [K][M], transB
// means B is stored [N][K].

// C = op(A) * op(B), plus colbias[col >> bias_shift] on every element when colbias is given.  Returns
// *biased = false when the shape took a kernel without that epilogue (the caller adds the bias itself).
// What may ride in a product's epilogue besides the bias forms: a reluGrad mask (C = mask > 0 ? product : 0).
struct Extras {
    const float *mask = nullptr;
};

int sgemm_epilogue(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B, float *C,
                   const float *colbias, int bias_shift, const float *rowvec, int relu, bool *biased, const Extras &ex = Extras{});

int sgemm_bias(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B, float *C,
               const float *colbias, int bias_shift, bool *biased)
{
    return sgemm_epilogue(transA, transB, M, N, K, A, B, C, colbias, bias_shift, nullptr, 0, biased);
}

// Which kernel a product takes and how it cuts the reduction: everything that decides the order in which an
// element's K terms are added.  It follows from the dimensions and the transposition flags alone - not from an epilogue
// being asked for, which a kernel without one leaves to a pass behind it; operand alignment picks between variants of a
// kernel that add in the same order (the LDS-resident kernel apart: panel_allowed = false is the route without it).
struct Route {
    enum Kind { kNone, kOuter, kGemvRows, kGemvColsShort, kGemvCols, kPanel, kSmall, kTile64, kTile128, kRows } kind;
    size_t cuts;    // partial sums per element that a second pass adds (gemv slices, tile-engine splits)
    size_t depth;   // reduction steps per partial sum (k per slice, slabs per split)
};

Route sgemm_route(int transA, int transB, size_t M, size_t N, size_t K, bool panel_allowed = true)
{
    Route r{Route::kNone, 1, K};
    if (M * N == 0 || K == 0) return r;
    if (K == 1) { r.kind = Route::kOuter; return r; }
    // matrix-vector products: `rows` reads the matrix row by row (k contiguous), `cols` column-wise
    if ((N == 1 && !transA) || (M == 1 && transB)) { r.kind = Route::kGemvRows; return r; }
    if ((M == 1 && !transB) || (N == 1 && transA)) {
        const size_t R = M == 1 ? N : M;
        if (K <= 256 && R < ((size_t)1 << 30)) { r.kind = Route::kGemvColsShort; return r; }   // one launch, no partial sums
        const size_t nblocks = ceil_div(R, (size_t)256);
        size_t slices = ceil_div((size_t)num_cus() * 2, nblocks);
        if (slices > ceil_div(K, (size_t)32)) slices = ceil_div(K, (size_t)32);
        if (slices > 64) slices = 64;
        if (slices < 1) slices = 1;
        r.kind = Route::kGemvCols;
        r.depth = ceil_div(K, slices);
        r.cuts = ceil_div(K, r.depth);
        return r;
    }
    // short reduction, both operands k-major, enough 128 x 128 tiles to fill the machine (alignment is checked at the
    // launch: the plan's buffers and every tensor of the pool are aligned)
    if (transA && !transB && panel_allowed && panel_shape(M, N, K)) { r.kind = Route::kPanel; return r; }
    // small and medium outputs: one block per 32 x 32 tile, the reduction split over its wavefronts.
    // Each tile reads its own 32 rows of A and 32 columns of B, so the operand traffic grows with the
    // number of tiles: up to 256 MB of it (served by the L2) this beats the LDS-tiled engine below,
    // whose 128-wide tiles leave most CUs with one four-wavefront block (1024 x 1024 x 256: 11 against
    // 22 us; 2048 x 2048 x 128: 21 against 31 us); beyond that the tile engine's operand reuse wins.
    const size_t tiles32 = ceil_div(M, (size_t)32) * ceil_div(N, (size_t)32);
    if (tiles32 <= 4096 && tiles32 * 64 * K * sizeof(float) <= ((size_t)256 << 20) && M * K < ((size_t)1 << 29) &&
        K * N < ((size_t)1 << 29)) {   // (32-bit byte offsets into either operand)
        r.kind = Route::kSmall;
        return r;
    }
    const bool big = M > 64;
    const size_t BM = big ? 128 : 64, BN = big ? 128 : 256;
    const size_t tiles = ceil_div(M, BM) * ceil_div(N, BN);
    const size_t slabs_total = ceil_div(K, (size_t)BK);
    size_t want = ((size_t)2 * num_cus() + tiles - 1) / tiles;
    const size_t max_by_depth = slabs_total / 4 > 0 ? slabs_total / 4 : 1;
    size_t splits = want < max_by_depth ? want : max_by_depth;
    if (splits > 32) splits = 32;
    if (splits < 1) splits = 1;
    r.depth = (slabs_total + splits - 1) / splits;
    r.cuts = (slabs_total + r.depth - 1) / r.depth;
    // more than 64 rows: row-major LDS tiles (sgemm_rows_k) while byte offsets into either operand fit 32 bits
    r.kind = !big ? Route::kTile64 : M * K < ((size_t)1 << 29) && K * N < ((size_t)1 << 29) ? Route::kRows : Route::kTile128;
    return r;
}

// The products with an epilogue: + rowvec[row] * colbias[col >> bias_shift] (rowvec optional), then relu.
// *biased says whether the kernel that ran applied it; if not, C holds the plain product.
int sgemm_epilogue(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B, float *C,
                   const float *colbias, int bias_shift, const float *rowvec, int relu, bool *biased, const Extras &ex)
{
    *biased = false;
    if (M * N == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(C != nullptr, "dopt_hip_sgemm: C is null");
    DOPT_ENSURE_INIT();
    if (K == 0) return dopt_hip_memset(C, 0, M * N * sizeof(float));  // beta = 0
    DOPT_REQUIRE(A && B, "dopt_hip_sgemm: null operand");
    DOPT_REQUIRE(M < ((size_t)1 << 30) && N < ((size_t)1 << 30) && K < ((size_t)1 << 30) &&
                     M * N < ((size_t)1 << 40),
                 "dopt_hip_sgemm: dimensions too large");

    Route route = sgemm_route(transA, transB, M, N, K);
    if (route.kind == Route::kPanel && !panel_takes(M, N, K, A, B))   // operands off the 16-byte grid: as if it were not there
        route = sgemm_route(transA, transB, M, N, K, false);
    const Route::Kind kind = route.kind;
    if (kind == Route::kOuter) {  // vectors: a transposed vector is the same memory
        hipLaunchKernelGGL(outer_k, dim3(flat_grid(M * N)), dim3(256), 0, stream(), M, N, A, B, C);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    if (kind == Route::kGemvRows) {
        const size_t R = N == 1 ? M : N;
        const float *mat = N == 1 ? A : B, *vec = N == 1 ? B : A;
        hipLaunchKernelGGL(gemv_rows_k, dim3((unsigned)ceil_div(R, (size_t)4)), dim3(256), 0, stream(), R, K, mat, vec, C);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    if (kind == Route::kGemvColsShort || kind == Route::kGemvCols) {
        const size_t R = M == 1 ? N : M;
        const float *mat = M == 1 ? B : A, *vec = M == 1 ? A : B;
        if (kind == Route::kGemvColsShort) {
            hipLaunchKernelGGL(gemv_cols_short_k, dim3((unsigned)ceil_div(R, (size_t)64)), dim3(256), 0, stream(), (int)K, (int)R,
                               vec, mat, C);
            DOPT_LAUNCH_CHECK();
            return DOPT_HIP_OK;
        }
        const size_t nblocks = ceil_div(R, (size_t)256), slices = route.cuts, kslice = route.depth;
        float *partial = C;
        if (slices > 1) {
            partial = (float *)workspace(slices * R * sizeof(float));
            if (!partial) return DOPT_HIP_ERR_OOM;
        }
        hipLaunchKernelGGL(gemv_cols_k, dim3((unsigned)nblocks, (unsigned)slices), dim3(256), 0, stream(), K, R, kslice,
                           vec, mat, partial);
        DOPT_LAUNCH_CHECK();
        if (slices > 1) {
            hipLaunchKernelGGL(splitk_reduce_k, dim3(flat_grid(R)), dim3(256), 0, stream(), R, (int)slices, partial, C);
            DOPT_LAUNCH_CHECK();
        }
        return DOPT_HIP_OK;
    }
    if (kind == Route::kPanel) return panel_launch(false, M, N, K, A, B, C);
    if (kind == Route::kSmall) {
        const int lda = (int)(transA ? M : K), ldb = (int)(transB ? K : N);
        int kslice = (int)ceil_div(ceil_div(K, (size_t)kSmallWaves), (size_t)8) * 8;
        // 128-bit loads for a k-contiguous operand whose rows start on 16-byte boundaries
        const bool va = !transA && aligned16(A) && lda % 4 == 0, vb = transB && aligned16(B) && ldb % 4 == 0;
        const dim3 grid((unsigned)ceil_div(N, (size_t)32), (unsigned)ceil_div(M, (size_t)32)), block(64 * kSmallWaves);
#define DOPT_SMALL(TA, TB, VA, VB)                                                                                       \
    hipLaunchKernelGGL((sgemm_small_k<TA, TB, VA, VB>), grid, block, 0, stream(), (int)M, (int)N, (int)K, lda, ldb, kslice, \
                       A, B, C, colbias, bias_shift, rowvec, relu, ex.mask)
        if (transA && transB) { if (vb) DOPT_SMALL(true, true, false, true); else DOPT_SMALL(true, true, false, false); }
        else if (transA) DOPT_SMALL(true, false, false, false);
        else if (transB) {
            if (va && vb) DOPT_SMALL(false, true, true, true);
            else if (va) DOPT_SMALL(false, true, true, false);
            else if (vb) DOPT_SMALL(false, true, false, true);
            else DOPT_SMALL(false, true, false, false);
        } else { if (va) DOPT_SMALL(false, false, true, false); else DOPT_SMALL(false, false, false, false); }
#undef DOPT_SMALL
        DOPT_LAUNCH_CHECK();
        *biased = true;   // whatever epilogue was asked for (the extras included), this kernel applied it
        return DOPT_HIP_OK;
    }

    Gemm g{};
    g.A = A;
    g.B = B;
    g.M = (int)M;
    g.N = (int)N;
    g.K = (int)K;
    g.lda = (int)(transA ? M : K);
    g.ldb = (int)(transB ? K : N);
    g.out_elems = M * N;
    g.slabs_total = (int)ceil_div(K, (size_t)BK);
    const bool big = kind != Route::kTile64;
    const int BM = big ? 128 : 64, BN = big ? 128 : 256;
    g.mtiles = (int)ceil_div(M, (size_t)BM);
    g.ntiles = (int)ceil_div(N, (size_t)BN);
    const int tiles = g.mtiles * g.ntiles;
    const int splits = (int)route.cuts;
    g.slabs_per_split = (int)route.depth;
    g.splits = splits;
    float *partial = nullptr;
    if (splits > 1) {
        partial = (float *)workspace((size_t)splits * g.out_elems * sizeof(float));
        if (!partial) return DOPT_HIP_ERR_OOM;
    }
    g.C = splits > 1 ? partial : C;
    // 128-bit loads for the operands stored with M (or N) contiguous
    const bool vec = (!transA || (M % 4 == 0 && aligned16(A))) && (transB || (N % 4 == 0 && aligned16(B)));
    dim3 grid(xcd_grid((unsigned)(tiles * splits)));
#define DOPT_SGEMM(BMV, TA, TB)                                                                               \
    do {                                                                                                      \
        if (vec) hipLaunchKernelGGL((sgemm_k<BMV, TA, TB, true>), grid, dim3(kGemmThreads), 0, stream(), g);   \
        else hipLaunchKernelGGL((sgemm_k<BMV, TA, TB, false>), grid, dim3(kGemmThreads), 0, stream(), g);      \
    } while (0)
#define DOPT_SGEMM_T(BMV)                                   \
    do {                                                    \
        if (!transA && !transB) DOPT_SGEMM(BMV, false, false); \
        else if (!transA) DOPT_SGEMM(BMV, false, true);     \
        else if (!transB) DOPT_SGEMM(BMV, true, false);     \
        else DOPT_SGEMM(BMV, true, true);                   \
    } while (0)
    // more than 64 rows: row-major LDS tiles (sgemm_rows_k)
    g.quads_a = g.lda % 4 == 0 && K % 4 == 0 && aligned16(A);
    g.quads_b = g.ldb % 4 == 0 && K % 4 == 0 && aligned16(B);
    if (kind == Route::kRows) {
#define DOPT_ROWS(TA, TB, QA, QB) hipLaunchKernelGGL((sgemm_rows_k<TA, TB, QA, QB>), grid, dim3(kGemmThreads), 0, stream(), g)
        const bool qa = g.quads_a, qb = g.quads_b;   // only a k-contiguous operand has the choice
        if (!transA && !transB) { if (qa) DOPT_ROWS(false, false, true, false); else DOPT_ROWS(false, false, false, false); }
        else if (!transA) {
            if (qa && qb) DOPT_ROWS(false, true, true, true);
            else if (qa) DOPT_ROWS(false, true, true, false);
            else if (qb) DOPT_ROWS(false, true, false, true);
            else DOPT_ROWS(false, true, false, false);
        } else if (!transB) DOPT_ROWS(true, false, false, false);
        else { if (qb) DOPT_ROWS(true, true, false, true); else DOPT_ROWS(true, true, false, false); }
#undef DOPT_ROWS
    } else if (big) DOPT_SGEMM_T(128);
    else DOPT_SGEMM_T(64);
#undef DOPT_SGEMM_T
#undef DOPT_SGEMM
    DOPT_LAUNCH_CHECK();
    if (splits > 1) {
        hipLaunchKernelGGL(splitk_reduce_k, dim3(flat_grid(g.out_elems)), dim3(256), 0, stream(), g.out_elems, splits,
                           partial, C);
        DOPT_LAUNCH_CHECK();
    }
    return DOPT_HIP_OK;
}

// Filter gradient of a 3x3, pad-1, unit-stride convolution over 2x2 images in one launch:
// dw[K][C][3][3] from x[N][4C] and dy[N][4K].  Returns false (nothing launched) when the shape does
// not suit the LDS-resident kernel; the caller then takes the product and folds it itself.
bool sgemm_fold2x2(size_t C, size_t K, size_t N, const float *x, const float *dy, float *dw, int *rc)
{
    if (!panel_takes(4 * C, 4 * K, N, x, dy)) return false;
    *rc = panel_launch(true, 4 * C, 4 * K, N, x, dy, dw);
    return true;
}

// The same for `n` layers at once (n <= 8): one launch when every layer suits the LDS-resident kernel, else false with
// nothing launched.
bool sgemm_fold2x2_batch(int n, const size_t *C, const size_t *K, const size_t *N, const float *const *x,
                         const float *const *dy, float *const *dw, int *rc)
{
    if (n < 1 || n > kGroupJobs) return false;
    size_t M4[kGroupJobs], N4[kGroupJobs];
    for (int i = 0; i < n; i++) {
        if (!panel_takes(4 * C[i], 4 * K[i], N[i], x[i], dy[i])) return false;
        M4[i] = 4 * C[i];
        N4[i] = 4 * K[i];
    }
    *rc = panel_fold_group_launch(n, M4, N4, N, x, dy, dw);
    return true;
}

}  // namespace dopt

extern "C" {

int dopt_hip_sgemm_batch(int n, const int *transA, const int *transB, const size_t *M, const size_t *N, const size_t *K,
                         const float *const *A, const float *const *B, float *const *C)
{
    using namespace dopt;
    DOPT_REQUIRE(n >= 0 && (n == 0 || (transA && transB && M && N && K && A && B && C)), "dopt_hip_sgemm_batch: null argument");
    DOPT_ENSURE_INIT();
    // Products that take the 32 x 32-tile kernel (grouped per template instance) or the short column sum share launches;
    // the others run one by one.  Outputs must not overlap any operand of the batch: the order inside it is not kept.
    struct Inst { bool ta, tb, va, vb; SmallGroup g; unsigned blocks; bool used; };
    std::vector<Inst> insts;
    std::vector<GemvJob> gemvs;
    std::vector<int> single;
    for (int i = 0; i < n; i++) {
        if (M[i] * N[i] == 0) continue;
        const bool plain = K[i] > 0 && A[i] && B[i] && C[i] && M[i] < ((size_t)1 << 30) && N[i] < ((size_t)1 << 30) && K[i] < ((size_t)1 << 30);
        const Route r = plain ? sgemm_route(transA[i], transB[i], M[i], N[i], K[i]) : Route{Route::kNone, 1, 0};
        if (r.kind == Route::kGemvColsShort && gemvs.size() < (size_t)kGroupJobs) {
            const size_t R = M[i] == 1 ? N[i] : M[i];
            GemvJob q{};
            q.K = (int)K[i]; q.N = (int)R;
            q.a = M[i] == 1 ? A[i] : B[i];
            q.B = M[i] == 1 ? B[i] : A[i];
            q.c = C[i];
            gemvs.push_back(q);
        } else if (r.kind == Route::kSmall) {
            const int lda = (int)(transA[i] ? M[i] : K[i]), ldb = (int)(transB[i] ? K[i] : N[i]);
            const bool ta = transA[i] != 0, tb = transB[i] != 0;
            const bool va = !ta && aligned16(A[i]) && lda % 4 == 0, vb = tb && aligned16(B[i]) && ldb % 4 == 0;
            // the instance the product would take alone (flags an instance does not read are false there)
            const bool iva = ta ? false : va, ivb = tb ? vb : false;
            Inst *in = nullptr;
            for (Inst &c : insts)
                if (c.ta == ta && c.tb == tb && c.va == iva && c.vb == ivb && c.g.ns < kGroupJobs) in = &c;
            if (!in) {
                insts.push_back(Inst{ta, tb, iva, ivb, SmallGroup{}, 0, false});
                in = &insts.back();
            }
            SmallJob &q = in->g.s[in->g.ns++];
            q.M = (int)M[i]; q.N = (int)N[i]; q.K = (int)K[i]; q.lda = lda; q.ldb = ldb;
            q.kslice = (int)ceil_div(ceil_div(K[i], (size_t)kSmallWaves), (size_t)8) * 8;
            q.nx = (int)ceil_div(N[i], (size_t)32);
            q.first = (int)in->blocks;
            q.A = A[i]; q.B = B[i]; q.C = C[i];
            in->blocks += (unsigned)(q.nx * ceil_div(M[i], (size_t)32));
        } else {
            single.push_back(i);
        }
    }
    for (size_t k = 0; k < insts.size(); k++) {
        Inst &in = insts[k];
        if (k == 0) {   // the column sums ride in the first launch
            for (const GemvJob &v : gemvs) {
                GemvJob &q = in.g.v[in.g.nv++];
                q = v;
                q.first = (int)in.blocks;
                in.blocks += (unsigned)ceil_div((size_t)v.N, (size_t)64);
            }
            gemvs.clear();
        }
        const dim3 grid(in.blocks), block(64 * kSmallWaves);
#define DOPT_GROUP(TA, TB, VA, VB) hipLaunchKernelGGL((sgemm_small_group_k<TA, TB, VA, VB>), grid, block, 0, stream(), in.g)
        if (in.ta && in.tb) { if (in.vb) DOPT_GROUP(true, true, false, true); else DOPT_GROUP(true, true, false, false); }
        else if (in.ta) DOPT_GROUP(true, false, false, false);
        else if (in.tb) {
            if (in.va && in.vb) DOPT_GROUP(false, true, true, true);
            else if (in.va) DOPT_GROUP(false, true, true, false);
            else if (in.vb) DOPT_GROUP(false, true, false, true);
            else DOPT_GROUP(false, true, false, false);
        } else { if (in.va) DOPT_GROUP(false, false, true, false); else DOPT_GROUP(false, false, false, false); }
#undef DOPT_GROUP
        DOPT_LAUNCH_CHECK();
    }
    for (const GemvJob &v : gemvs) {   // no 32 x 32-tile launch to ride in
        hipLaunchKernelGGL(gemv_cols_short_k, dim3((unsigned)ceil_div((size_t)v.N, (size_t)64)), dim3(256), 0, stream(), v.K, v.N,
                           v.a, v.B, v.c);
        DOPT_LAUNCH_CHECK();
    }
    for (int i : single)
        if (int rc = dopt_hip_sgemm_t(transA[i], transB[i], M[i], N[i], K[i], A[i], B[i], C[i])) return rc;
    return DOPT_HIP_OK;
}

int dopt_hip_sgemm_rank1(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B,
                         const float *u, const float *v, int relu, float *C)
{
    DOPT_REQUIRE((u == nullptr) == (v == nullptr), "dopt_hip_sgemm_rank1: u and v go together");
    bool applied = false;
    if (int rc = dopt::sgemm_epilogue(transA, transB, M, N, K, A, B, C, v, 0, u, relu, &applied)) return rc;
    if (applied || M * N == 0 || (!v && !relu)) return DOPT_HIP_OK;
    hipLaunchKernelGGL(rank1_epilogue_k, dim3(flat_grid(M * N)), dim3(256), 0, dopt::stream(), M, N, u, v, relu, C);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_sgemm_relu_grad(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B,
                             const float *x, float *C)
{
    DOPT_REQUIRE(x != nullptr || M * N == 0, "dopt_hip_sgemm_relu_grad: null argument");
    dopt::Extras ex;
    ex.mask = x;
    bool applied = false;
    if (int rc = dopt::sgemm_epilogue(transA, transB, M, N, K, A, B, C, nullptr, 0, nullptr, 0, &applied, ex)) return rc;
    if (applied || M * N == 0) return DOPT_HIP_OK;
    return dopt_hip_relu_bwd(M * N, C, x, C);   // in place: every element is read before it is written
}

uint64_t dopt_hip_sgemm_order(int transA, int transB, size_t M, size_t N, size_t K)
{
    if (!dopt::ensure_init()) return 0;   // the cut of a reduction follows the device's size
    const dopt::Route r = dopt::sgemm_route(transA, transB, M, N, K);
    return (uint64_t)r.kind | (uint64_t)r.cuts << 8 | (uint64_t)r.depth << 24;
}

int dopt_hip_sgemm_t(int transA, int transB, size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    bool biased;
    return dopt::sgemm_bias(transA, transB, M, N, K, A, B, C, nullptr, 0, &biased);
}

int dopt_hip_sgemm(size_t M, size_t N, size_t K, const float *A, const float *B, float *C)
{
    return dopt_hip_sgemm_t(0, 0, M, N, K, A, B, C);
}

}  // extern "C"
