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
// channels differ by a wave-uniform offset.  Wp is the filter re-packed once per call into
// [tap*ci][m] (m contiguous), so the A tile goes global -> LDS with 128-bit accesses.
//
// Backward-filter is a GEMM with M = K (output channels), columns = (r', s', c) tap-major with c
// padded to 16, reduction = output pixels (n,p,q); both operands are gathered with lanes along
// the pixel index (contiguous in memory).  A second kernel sums the reduction splits and permutes
// the columns back to [K][C][R][S].
//
// All gathers go through buffer-resource loads whose range check supplies the zero padding, so
// the inner loops are branch-free.  Layers with few output tiles split the reduction; partial
// tiles go to the workspace and are summed in a fixed order -- no float atomics, so results are
// reproducible.
#include <utility>
#include <vector>

#include "common.h"
#include "mfma_core.h"

namespace {

using namespace dopt;

constexpr int BK = 16;

// ------------------------------------------------------------------------------------ gather

struct GatherConv {
    const float *in;   // gathered operand [N, Cin, IH, IW]
    const float *wp;   // packed filter [taps * CinPad][Mp]
    float *out;        // [N, Mout, OH, OW], or `splits` partial copies of it
    int N, Cin, IH, IW, Mout, OH, OW, R, S;
    int padH, padW, strideH, strideW;
    int CinPad, Mp, ncols;
    int mtiles, ntiles, slabs_total, slabs_per_split, splits;
    size_t out_elems, in_bytes, wp_bytes;
    // where output pixel (oh, ow) of this problem lands: row oh * out_sy + out_oy, column ow * out_sx +
    // out_ox of a plane of out_plane elements and out_OW columns (the whole tensor, or every
    // stride-th pixel of it when a strided backward-data pass is run class by class)
    int out_plane, out_OW, out_sy, out_sx, out_oy, out_ox;
};

// kMode: 0 = forward, 1 = backward-data with unit stride (no divisions), 2 = backward-data, any stride.
// L: the workgroup's item among the problem's (split, tile) pairs, tile fastest.
template <class T, int kMode>
__device__ __forceinline__ void conv_gather_body(const GatherConv &p, unsigned L)
{
    constexpr int BM = T::BM, BN = T::BN, LDA = T::LDA, LDB = T::LDB, THREADS = T::THREADS;
    constexpr int NA = BM * BK / 4 / THREADS;  // float4 loads of A per thread
    constexpr int RSTEP = THREADS / BN;        // reduction rows covered by one pass of B loads
    constexpr int NB = BK / RSTEP;             // scalar loads of B per thread
    static_assert(NA >= 1 && NB >= 1 && RSTEP >= 1, "tile too small for the thread count");
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int slab_begin = split * p.slabs_per_split;
    const int slab_end = min(slab_begin + p.slabs_per_split, p.slabs_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / T::WN, wn = w % T::WN;

    const __amdgpu_buffer_rsrc_t rin = make_rsrc(p.in, p.in_bytes);
    const __amdgpu_buffer_rsrc_t rwp = make_rsrc(p.wp, p.wp_bytes);

    // A: this thread's float4 slots of the [BK][BM] filter tile; byte offset relative to the slab's first row
    unsigned a_voff[NA];
    int a_lds[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) {
        const int f = tid + THREADS * i;
        const int row = f / (BM / 4), gm = m0 + (f % (BM / 4)) * 4;
        a_voff[i] = gm < p.Mp ? (unsigned)(row * p.Mp + gm) * 4u : kOobOffset;
        a_lds[i] = row * LDA + (f % (BM / 4)) * 4;
    }

    // B: the output pixel this thread gathers for
    const int bcol = tid % BN, brow0 = tid / BN;
    const int pix = n0 + bcol;
    const int pix_oob = p.ncols - 1 - pix;  // negative past the last pixel
    const int OHW = p.OH * p.OW;
    const int n_img = pix / OHW, pq = pix - n_img * OHW;
    const int oh = pq / p.OW, ow = pq - oh * p.OW;
    const int chan_stride = p.IH * p.IW;
    const int pix_base = (n_img * p.Cin + brow0) * chan_stride;  // element offset of (n, channel brow0, 0, 0)
    const int row_limit = p.Cin - brow0;                          // rows with ci0 + RSTEP*i >= row_limit are padding
    const bool c_full = p.CinPad == p.Cin;

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
        int ih, iw, bad = pix_oob;
        if (kMode == 0) {
            ih = oh * p.strideH - p.padH + (p.R - 1 - tr);
            iw = ow * p.strideW - p.padW + (p.S - 1 - ts);
        } else if (kMode == 1) {
            ih = oh + p.padH - (p.R - 1 - tr);
            iw = ow + p.padW - (p.S - 1 - ts);
        } else {
            // out = dx[.., h, w]; in = dy[.., ph, qw] with h = ph*stride - pad + r, r = R-1-tr
            const int nh = oh + p.padH - (p.R - 1 - tr), nw = ow + p.padW - (p.S - 1 - ts);
            ih = nh / p.strideH;
            iw = nw / p.strideW;
            // negative numerators, and numerators that are not multiples of the stride, hit no input
            bad |= nh | nw | -(int)(ih * p.strideH != nh) | -(int)(iw * p.strideW != nw);
        }
        bad |= ih | (p.IH - 1 - ih) | iw | (p.IW - 1 - iw);  // sign bit set: outside the input
        const unsigned b_voff = bad < 0 ? kOobOffset : (unsigned)(pix_base + ih * p.IW + iw) * 4u;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int ci = ci0 + RSTEP * i;  // wave-uniform
            const unsigned voff = (c_full || ci < row_limit) ? b_voff : kOobOffset;
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

    v16f acc[T::MI][T::NI];
    zero_acc(acc);
    load();
    store(0);
    __syncthreads();
    int cur = 0;
    // steady state: no data-dependent branches inside
    for (int slab = slab_begin; slab < slab_end - 1; ++slab) {
        load();
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * (BM / T::WM), wn * (BN / T::WN), acc, lane);
        store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * (BM / T::WM), wn * (BN / T::WN), acc, lane);

    float *outp = p.out + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < T::NI; j++) {
        const int col = n0 + wn * (BN / T::WN) + j * 32 + (lane & 31);
        if (col >= p.ncols) continue;
        const int n2 = col / OHW, pq2 = col - n2 * OHW;
        const int oh2 = pq2 / p.OW, ow2 = pq2 - oh2 * p.OW;
        float *base = outp + (size_t)n2 * p.Mout * p.out_plane + (size_t)(oh2 * p.out_sy + p.out_oy) * p.out_OW +
                      ow2 * p.out_sx + p.out_ox;
#pragma unroll
        for (int i = 0; i < T::MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * (BM / T::WM) + i * 32 + acc_row(v, lane);
                if (m < p.Mout) base[(size_t)m * p.out_plane] = acc[i][j][v];
            }
    }
}

template <class T, int kMode>
__global__ __launch_bounds__(T::THREADS, T::THREADS / 128) void conv_gather_k(GatherConv p)
{
    // 1-D grid over (split, tile), tile fastest: the blocks an XCD receives work on neighbouring
    // tiles of the same slice of the reduction, whatever the ratio of tiles to splits
    unsigned L;
    if (!xcd_remap(blockIdx.x, (unsigned)(p.mtiles * p.ntiles) * (unsigned)p.splits, &L)) return;
    conv_gather_body<T, kMode>(p, L);
}

// Up to nine problems that do not depend on each other in ONE launch (the residue classes of a strided backward-data
// pass - four at stride 2, nine at stride 3: same operands, different sub-filters, interleaved output pixels).  Every workgroup runs conv_gather_body on one
// tile of one problem, so each problem's values are those of a launch of its own; what changes is that the chip is not
// drained and refilled between problems that each fill only part of it.  An XCD takes the same share of every problem
// (its tiles of a problem are neighbours, as in a single launch), longest problem first.
constexpr int kGatherJobs = 9;
struct GatherGroup {
    GatherConv g[kGatherJobs];
    unsigned per[kGatherJobs];   // workgroups of problem j on each XCD: ceil(tiles * splits / 8)
    int n;
};

template <class T, int kMode>
__global__ __launch_bounds__(T::THREADS, T::THREADS / 128) void conv_gather_group_k(GatherGroup gg)
{
    const unsigned xcd = blockIdx.x & 7u;
    unsigned i = blockIdx.x >> 3;
    int j = 0;
    while (j < gg.n - 1 && i >= gg.per[j]) {
        i -= gg.per[j];
        j++;
    }
    const unsigned L = xcd * gg.per[j] + i;
    if (i >= gg.per[j] || L >= (unsigned)(gg.g[j].mtiles * gg.g[j].ntiles) * (unsigned)gg.g[j].splits) return;
    conv_gather_body<T, kMode>(gg.g[j], L);
}

// ------------------------------------------------------------------------------------ patch (3x3, unit stride)
//
// Forward and backward-data of 3x3 unit-stride convolutions.  The gathered operand is not
// re-fetched per filter tap: for a chunk of 16 input channels the block loads the input patch
// under its pixel tile ONCE -- the tile's rows plus a one-pixel halo, zero-filled outside the
// image by the buffer range check -- and the nine taps read it at nine offsets.  LDS holds the
// patch position-major, Bp[pos][16 channels (+4 pad)], so that a lane's pixel operands for a whole
// 16-channel slab are two 128-bit LDS reads per 32-wide fragment; the packed filter,
// wp[slab][m][16 channels], has the same shape per row, and a lane's filter operands are two 128-bit
// loads straight from it.  Lane half kh (= lane / 32) multiplies channels kh*8 .. kh*8+7 of the
// chunk over the slab's eight matrix steps (the same channel permutation on both operands, so
// every channel is counted once).  Per 32 matrix instructions a wavefront issues 4 patch fragment
// reads, 4 filter loads and ~5 patch loads and stores.

struct PatchConv {
    const float *in;   // gathered operand [N, Cin, IH, IW]
    const float *wp;   // packed filter [chunks][9][Mp][16]
    float *out;        // [N, Mout, OH, OW], or `splits` partial copies of it
    const float *bias; // optional [Mout], added to the finished sums (by the split reduction when there is one)
    int N, Cin, IH, IW, Mout, OH, OW;
    int PT, PL;        // input row / column of patch position (0,0) is (oh0 - PT, -PL)
    int flip;          // 1: tap (tr,ts) reads patch offset (2-tr, 2-ts); 0: (tr, ts)
    int nimg, rows;    // images per pixel tile; output rows of each image in the tile
    int PR, PC, psz;   // patch rows and columns per image; patch positions per tile = nimg*PR*PC
    unsigned magic_psz, magic_img, magic_pc;  // floor(2^32/d)+1 for d = psz, PR*PC, PC (exact for x*d < 2^32)
    int Mp;            // rows of one packed filter slab (Mout rounded up to the tile height)
    int ncols, mtiles, ntiles, chunks_total, chunks_per_split, splits;
    size_t out_elems, in_bytes, wp_bytes;
};

__device__ inline unsigned fast_div(unsigned x, unsigned magic) { return __umulhi(x, magic); }

// The filter fragments go from memory straight into the registers the matrix cores read: the
// packed layout is the fragment layout (a wavefront fetches 32 rows x 64 bytes, 2 KB contiguous, per
// 32 output channels and tap; the four wavefronts of a tile row fetch the same lines, three of them
// from the L1), one tap ahead.  Only the patch goes through LDS, double buffered, so the workgroup
// meets once per 16-channel chunk, when the patch buffers swap.  (Staging the filter slab in LDS as
// well costs a barrier per tap: 1.1 % slower on the VGG step.)
template <class T, int NPMAX, bool kCFull>
__device__ __forceinline__ void conv_patch_body(const PatchConv &p, const unsigned block_id)
{
    constexpr int BM = T::BM, BN = T::BN, THREADS = T::THREADS, MI = T::MI, NI = T::NI;
    constexpr int TAPS = 9, CH = 16, LDP = 20;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int pstride = (p.psz + 1) * LDP;  // one spare position absorbs the stores of unused slots
    float *const Bp0 = lds;                  // [2][pstride]

    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    if (!xcd_remap(block_id, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int cb = split * p.chunks_per_split;
    const int ce = min(cb + p.chunks_per_split, p.chunks_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int wm = w / T::WN, wn = w % T::WN;
    const int kh = lane >> 5, l32 = lane & 31;
    const int OHW = p.OH * p.OW;
    const int chan_stride = p.IH * p.IW;

    const __amdgpu_buffer_rsrc_t rin = make_rsrc(p.in, p.in_bytes);
    const __amdgpu_buffer_rsrc_t rwp = make_rsrc(p.wp, p.wp_bytes);

    // ---- patch slots of this thread: element e = i*THREADS + tid -> (channel e / psz, position e % psz)
    const int n_first = n0 / OHW, oh0 = (n0 - n_first * OHW) / p.OW;
    unsigned p_voff[NPMAX];  // byte offset of the element inside channel chunk 0, or kOobOffset
    int p_lds[NPMAX];        // byte offset inside a patch buffer
    int p_chan[NPMAX];       // channel inside the chunk (only read when the last chunk is ragged)
#pragma unroll
    for (int i = 0; i < NPMAX; i++) {
        const unsigned e = (unsigned)(i * THREADS + tid);
        const unsigned c = fast_div(e, p.magic_psz);
        const unsigned pos = e - c * (unsigned)p.psz;
        const unsigned img = fast_div(pos, p.magic_img);
        const unsigned rem = pos - img * (unsigned)(p.PR * p.PC);
        const unsigned pr = fast_div(rem, p.magic_pc);
        const unsigned pc = rem - pr * (unsigned)p.PC;
        const int n = n_first + (int)img, ih = oh0 + (int)pr - p.PT, iw = (int)pc - p.PL;
        const int bad = (CH - 1 - (int)c) | (p.N - 1 - n) | ih | (p.IH - 1 - ih) | iw | (p.IW - 1 - iw);
        p_voff[i] = bad < 0 ? kOobOffset : (unsigned)(((n * p.Cin + (int)c) * p.IH + ih) * p.IW + iw) * 4u;
        p_lds[i] = c < (unsigned)CH ? (int)(pos * LDP + c) * 4 : (p.psz * LDP + (tid & 15)) * 4;
        p_chan[i] = (int)c;
    }
    float preg[NPMAX];
    auto patch_load = [&](int i, int chunk) {
        unsigned voff = p_voff[i];
        if (!kCFull) voff = chunk * CH + p_chan[i] < p.Cin ? voff : kOobOffset;
        preg[i] = buffer_load_f32(rin, voff, (unsigned)(chunk * CH * chan_stride) * 4u);
    };
    auto patch_store = [&](int i, float *buf) { *(float *)((char *)buf + p_lds[i]) = preg[i]; };

    // ---- filter fragments: this lane's 8 channels (kh * 8 ..) of row l32 of each 32-row group
    const unsigned slab_bytes = (unsigned)p.Mp * CH * 4u;
    const unsigned fa_voff = (unsigned)((m0 + wm * (BM / T::WM) + l32) * CH + kh * 8) * 4u;   // m0 + row < Mp always
    // three sets of filter fragments: the tap being multiplied, the next one, and the one after it on its way (a tap
    // lasts ~0.4 us per wavefront, less than a load from the L2 can take under load)
    float4 fa_ring[3][MI][2];
    auto fa_load = [&](auto slot_tag, int slab) {   // past the last slab the range check returns zeros
        constexpr int slot = decltype(slot_tag)::value;
#pragma unroll
        for (int i = 0; i < MI; i++) {
            fa_ring[slot][i][0] = buffer_load_f32x4(rwp, fa_voff + (unsigned)(i * 32 * CH) * 4u, (unsigned)slab * slab_bytes);
            fa_ring[slot][i][1] = buffer_load_f32x4(rwp, fa_voff + (unsigned)(i * 32 * CH) * 4u + 16u, (unsigned)slab * slab_bytes);
        }
    };
    int b_frag[NI];  // float offset inside a patch buffer of this lane's pixel, tap offset (0,0)
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int q = wn * (BN / T::WN) + j * 32 + l32;  // pixel inside the tile
        const int img = q / (p.rows * p.OW), r = q / p.OW - img * p.rows, col = q % p.OW;
        b_frag[j] = ((img * p.PR + r) * p.PC + col) * LDP + kh * 8;
    }

    v16f acc[MI][NI];
    zero_acc(acc);

    // prologue: the first patch and the first filter slab
#pragma unroll
    for (int i = 0; i < NPMAX; i++) patch_load(i, cb);
    fa_load(StepTag<0>{}, cb * TAPS);
    fa_load(StepTag<1>{}, cb * TAPS + 1);
#pragma unroll
    for (int i = 0; i < NPMAX; i++) patch_store(i, Bp0);
    __syncthreads();

    int pcur = 0;
    int sidx = cb * TAPS;  // filter slab being multiplied
    // loads of the next patch are issued during taps 0..3 of a chunk, its LDS stores during taps 5..8
    constexpr int PER = (NPMAX + 3) / 4;
    for (int chunk = cb; chunk < ce; ++chunk) {
        float *const bp_cur = Bp0 + pcur * pstride;
        float *const bp_nxt = Bp0 + (pcur ^ 1) * pstride;
        static_for<0, TAPS>([&](auto ttag) {
            constexpr int t = decltype(ttag)::value;
            constexpr int tr = t / 3, ts = t % 3;
            const int tapoff = (p.flip ? (2 - tr) * p.PC + (2 - ts) : tr * p.PC + ts) * LDP;
            float4 fa[MI][2], fb[NI][2];
#pragma unroll
            for (int i = 0; i < MI; i++) {   // nine taps per chunk: the ring slot of a tap is the same in every chunk
                fa[i][0] = fa_ring[t % 3][i][0];
                fa[i][1] = fa_ring[t % 3][i][1];
            }
#pragma unroll
            for (int j = 0; j < NI; j++) {
                fb[j][0] = *(const float4 *)(bp_cur + b_frag[j] + tapoff);
                fb[j][1] = *(const float4 *)(bp_cur + b_frag[j] + tapoff + 4);
            }
            static_for<0, 8>([&](auto stag) {
                constexpr int ks = decltype(stag)::value;
                // side work of this step
                if constexpr (ks == 0) fa_load(StepTag<(t + 2) % 3>{}, sidx + 2);
                if constexpr (t < 4 && ks >= 1 && ks <= 6) {
                    // PER loads of tap t, dealt over steps 1..6
                    constexpr int first = t * PER + (ks - 1) * ((PER + 5) / 6);
                    constexpr int last = first + (PER + 5) / 6;
#pragma unroll
                    for (int i = first; i < last; i++)
                        if (i < (t + 1) * PER && i < NPMAX) patch_load(i, chunk + 1);
                }
                if constexpr (t >= 5 && ks >= 1 && ks <= 6) {
                    constexpr int first = (t - 5) * PER + (ks - 1) * ((PER + 5) / 6);
                    constexpr int last = first + (PER + 5) / 6;
#pragma unroll
                    for (int i = first; i < last; i++)
                        if (i < (t - 4) * PER && i < NPMAX) patch_store(i, bp_nxt);
                }
#pragma unroll
                for (int i = 0; i < MI; i++)
#pragma unroll
                    for (int j = 0; j < NI; j++) {
                        const float4 av = fa[i][ks / 4], bv = fb[j][ks / 4];
                        const float a = ks % 4 == 0 ? av.x : ks % 4 == 1 ? av.y : ks % 4 == 2 ? av.z : av.w;
                        const float b = ks % 4 == 0 ? bv.x : ks % 4 == 1 ? bv.y : ks % 4 == 2 ? bv.z : bv.w;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i][j], 0, 0, 0);
                    }
#pragma unroll
                for (int g = 0; g < MI * NI; g++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x216, 2, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (t == TAPS - 1) __syncthreads();
            ++sidx;
        });
        pcur ^= 1;
    }

    float *outp = p.out + (size_t)split * p.out_elems;
    const bool add_bias = p.bias != nullptr && p.splits == 1;
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int col = n0 + wn * (BN / T::WN) + j * 32 + l32;
        if (col >= p.ncols) continue;
        const int n2 = col / OHW, pq2 = col - n2 * OHW;
        float *base = outp + (size_t)n2 * p.Mout * OHW + pq2;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * (BM / T::WM) + i * 32 + acc_row(v, lane);
                if (m < p.Mout) base[(size_t)m * OHW] = add_bias ? acc[i][j][v] + p.bias[m] : acc[i][j][v];
            }
    }
}

template <class T, int NPMAX, bool kCFull>
__global__ __launch_bounds__(T::THREADS, T::THREADS / 256) void conv_patch_k(PatchConv p)
{
    conv_patch_body<T, NPMAX, kCFull>(p, blockIdx.x);
}

// ------------------------------------------------------------------------------------ Winograd F(2x2, 3x3)
//
// The same layers (3x3, unit stride, pad 1, even image sides, whole 16-channel chunks) with 16 instead of 36
// multiplications per 2x2 output pixels (Lavin & Gray): Y = At [ (G g Gt) . (Bt d B) ] A, the element-wise product summed
// over the channels - sixteen independent [rows x channels] . [channels x tiles] products, one per position xi of the
// 4x4 transformed tile.  The direct kernels run at three quarters of the fp32 matrix peak, so what is left to remove is
// arithmetic.
//
// A workgroup owns 128 rows x 32 tiles (the 128 pixels of the direct kernel's column tile: whole image rows or whole
// images, so the input under them is the same rectangle with the same zero halo) or 64 rows x 64 tiles.
// Per 16-channel chunk: the raw patch goes to LDS position-major (a thread owns one position and stores its channels
// as 128-bit pieces); all 512 threads transform it - thread (i, tile, four channels) forms row i of Bt d B for its tile
// from eight 128-bit reads and writes the four transformed values, four channels each, to V[xi][tile][16 channels];
// wavefront (wk, wi) multiplies rows 32 wk .. + 31 with the eight positions xi = 8 wi .. 8 wi + 7: per position two
// 128-bit reads of V (this lane's tile, its eight channels; one position ahead) and two 128-bit loads of the
// transformed filter U[chunk][xi][row][16 channels] straight into operand registers, three positions ahead, feed
// eight matrix instructions into the position's own accumulator (128 accumulator registers per wavefront, two
// wavefronts per SIMD).  With 32 tiles, patch and V are double-buffered and the next chunk's transform runs under
// this chunk's matrix instructions; every piece of side work is pinned to a matrix step (sched_barrier), or the
// scheduler sinks the prefetches to their first use.
//
// At the end a lane holds M[xi][row][tile] for its eight positions - two rows i of the 4x4 grid, complete in j - so it
// applies A along j in registers (z[i][b]), combines its two rows into its share of the four outputs, and the
// wavefronts of a pair add their shares through LDS: y[a][b] = (At z)[a][b].  Output, split reductions and bias are
// those of the direct kernel.
//
// What bounds it: a chunk is 3.4 us of matrix time per workgroup at the nominal rate, 3.95 in a build of this loop with
// nothing but its matrix instructions, and takes 4.6 .. 5.0 - the filter loads (128 KB per chunk
// and workgroup, 16/9 the direct kernel's), the V reads, the patch and the transform each add their share, roughly in
// proportion to their instruction counts (loops without one of them: -0.5, -0.2, -0.3, -0.4 us).  128 rows x 64 tiles
// would halve filter traffic and fragment loads per matrix instruction and need 256 accumulator registers per wavefront.
constexpr int kWinoXchg = 4 * 64 * 64;   // floats of the exchange area: four wavefront pairs x 64 values per lane

// WK x TH: the eight wavefronts are WK groups of 32 rows x TH groups of 32 tiles x the two halves of the 16 positions:
// 4 x 1 (128 rows x 32 tiles = 128 pixels) for layers with whole 128-row tiles, 2 x 2 (64 rows x 64 tiles = 256 pixels)
// for 64-row layers.
template <int NPMAX, int WK, int TH>
__global__ __launch_bounds__(512, 1) void conv_wino_k(PatchConv p)
{
    static_assert(WK * TH == 4 && NPMAX == 16, "eight wavefronts, sixteen channels per chunk");
    constexpr int BM = 32 * WK, BN = 128 * TH, TT = 32 * TH, CH = 16, LDP = 20, VSZ = 16 * TT * LDP;
    // 32 tiles per workgroup: V and the raw patch are double-buffered, the transform of the next chunk runs under this
    // chunk's matrix instructions and the workgroup meets once per chunk.  64 tiles: one V (80 KB), transformed between
    // two barriers.
    constexpr bool DB = TH == 1;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int raw_floats = ((p.psz + 1) * LDP + 3) / 4 * 4;   // one spare position absorbs the stores of idle threads
    float *const raw0 = lds;
    float *const V0 = lds + (DB ? 2 : 1) * raw_floats;          // [16][TT][LDP] (x 2)

    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ntiles);
    if (!xcd_remap(blockIdx.x, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), nt = (int)(tile / (unsigned)p.mtiles);
    const int m0 = mt * BM, n0 = nt * BN;
    const int cb = split * p.chunks_per_split;
    const int ce = min(cb + p.chunks_per_split, p.chunks_total);
    const int nch = ce - cb;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront-uniform, and known to be: it enters scalar load offsets
    const int wi = w & 1, wk = (w >> 1) % WK, th = (w >> 1) / WK;
    const int kh = lane >> 5, l32 = lane & 31;
    const int OHW = p.OH * p.OW;
    const int chan_stride = p.IH * p.IW;
    const __amdgpu_buffer_rsrc_t rin = make_rsrc(p.in, p.in_bytes);
    const __amdgpu_buffer_rsrc_t rwp = make_rsrc(p.wp, p.wp_bytes);

    // ---- the patch: a thread owns ONE position and loads `nslots` of the chunk's channels of it, so its sixteen
    // addresses are one per-lane offset plus a wavefront-uniform channel offset (sixteen separate offsets and LDS
    // addresses would hold 32 registers).  Up to 256 positions: wavefronts 4..7 take channels 8..15 of the same positions.
    const int n_first = n0 / OHW, oh0 = (n0 - n_first * OHW) / p.OW;
    const int nslots = p.psz <= 256 ? 8 : 16;
    const int pos = p.psz <= 256 ? (tid & 255) : tid;
    const int cbase = p.psz <= 256 ? (w >> 2) * 8 : 0;
    unsigned p_voff;
    int p_lds;
    {
        const unsigned ps = (unsigned)min(pos, p.psz - 1);
        const unsigned img = fast_div(ps, p.magic_img);
        const unsigned rem = ps - img * (unsigned)(p.PR * p.PC);
        const unsigned pr = fast_div(rem, p.magic_pc);
        const unsigned pc = rem - pr * (unsigned)p.PC;
        const int n = n_first + (int)img, ih = oh0 + (int)pr - p.PT, iw = (int)pc - p.PL;
        const int bad = (p.psz - 1 - pos) | (p.N - 1 - n) | ih | (p.IH - 1 - ih) | iw | (p.IW - 1 - iw);
        p_voff = bad < 0 ? kOobOffset : (unsigned)((n * p.Cin * p.IH + ih) * p.IW + iw) * 4u;
        p_lds = (min(pos, p.psz) * LDP + cbase) * 4;
    }
    float preg[NPMAX];
    auto patch_load = [&](int i, int chunk) {
        if (i < nslots) preg[i] = buffer_load_f32(rin, p_voff, (unsigned)((chunk * CH + cbase + i) * chan_stride) * 4u);
    };
    auto patch_store = [&](int g, float *rawb) {   // channels 4 g .. 4 g + 3 of the position: one 128-bit store
        if (4 * g < nslots)
            *(float4 *)((char *)rawb + p_lds + g * 16) = make_float4(preg[4 * g], preg[4 * g + 1], preg[4 * g + 2], preg[4 * g + 3]);
    };

    // ---- the transform items of this thread (TH of them): row ti of Bt d B for tile tau, channels 4 cq .. 4 cq + 3
    const int tcn = p.OW >> 1, tpi = (p.rows >> 1) * tcn;          // tiles per row of tiles, per image of the pixel tile
    // Bt = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]: row ti is d[ra] + sg * d[rb]
    int t_a[TH], t_b[TH], t_out[TH];
    float sg[TH];
#pragma unroll
    for (int u = 0; u < TH; u++) {
        const int item = u * 512 + tid, ti = item / (TT * 4), tau_t = (item % (TT * 4)) >> 2, cq = item & 3;
        const int img = tau_t / tpi, tl = tau_t - img * tpi, r2 = tl / tcn, c2 = tl - r2 * tcn;
        const int t_in = ((img * p.PR + 2 * r2) * p.PC + 2 * c2) * LDP + cq * 4;
        const int ra = ti == 0 ? 0 : ti == 2 ? 2 : 1, rb = ti == 0 ? 2 : ti == 1 ? 2 : ti == 2 ? 1 : 3;
        t_a[u] = t_in + ra * p.PC * LDP;
        t_b[u] = t_in + rb * p.PC * LDP;
        t_out[u] = ((ti * 4) * TT + tau_t) * LDP + cq * 4;
        sg[u] = ti == 1 ? 1.0f : -1.0f;
    }
    float4 tt[TH][4];
    auto transform_read = [&](int b, const float *rawb) {       // column b of the thread's row of Bt d
#pragma unroll
        for (int u = 0; u < TH; u++) {
            const float4 da = *(const float4 *)(rawb + t_a[u] + b * LDP), db = *(const float4 *)(rawb + t_b[u] + b * LDP);
            // sg is +-1: the fused form rounds once, like the sum or difference it stands for
            tt[u][b] = make_float4(__builtin_fmaf(sg[u], db.x, da.x), __builtin_fmaf(sg[u], db.y, da.y),
                                   __builtin_fmaf(sg[u], db.z, da.z), __builtin_fmaf(sg[u], db.w, da.w));
        }
    };
    auto transform_write = [&](float *Vb) {                      // ... times B: four positions, four channels each
        auto sub = [](float4 x, float4 y) { return make_float4(x.x - y.x, x.y - y.y, x.z - y.z, x.w - y.w); };
        auto add = [](float4 x, float4 y) { return make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w); };
#pragma unroll
        for (int u = 0; u < TH; u++) {
            *(float4 *)(Vb + t_out[u]) = sub(tt[u][0], tt[u][2]);
            *(float4 *)(Vb + t_out[u] + TT * LDP) = add(tt[u][1], tt[u][2]);
            *(float4 *)(Vb + t_out[u] + 2 * TT * LDP) = sub(tt[u][2], tt[u][1]);
            *(float4 *)(Vb + t_out[u] + 3 * TT * LDP) = sub(tt[u][1], tt[u][3]);
        }
    };

    // ---- transformed-filter fragments: this lane's 8 channels (kh * 8 ..) of row m0 + 32 wk + l32
    const unsigned slab_bytes = (unsigned)p.Mp * CH * 4u;
    const unsigned fa_voff = (unsigned)((m0 + wk * 32 + l32) * CH + kh * 8) * 4u;
    float4 fa_ring[4][2];
    auto fa_load = [&](auto slot_tag, int slab) {   // past the last slab the range check returns zeros
        constexpr int slot = decltype(slot_tag)::value;
        fa_ring[slot][0] = buffer_load_f32x4(rwp, fa_voff, (unsigned)slab * slab_bytes);
        fa_ring[slot][1] = buffer_load_f32x4(rwp, fa_voff + 16u, (unsigned)slab * slab_bytes);
    };
    const int b_frag = (wi * 8 * TT + th * 32 + l32) * LDP + kh * 8;   // position 8 wi, this lane's tile and channels

    v16f acc[8];
#pragma unroll
    for (int x = 0; x < 8; x++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[x][v] = 0.0f;

    // prologue: the first patch (and, double-buffered, the second: both in flight together), the first transform, the
    // first three filter fragments
#pragma unroll
    for (int i = 0; i < NPMAX; i++) patch_load(i, cb);
    if constexpr (DB) {
        float second[NPMAX];
#pragma unroll
        for (int i = 0; i < NPMAX; i++)
            second[i] = i < nslots && nch > 1 ? buffer_load_f32(rin, p_voff, (unsigned)(((cb + 1) * CH + cbase + i) * chan_stride) * 4u) : 0.0f;
        fa_load(StepTag<0>{}, cb * 16 + wi * 8);
        fa_load(StepTag<1>{}, cb * 16 + wi * 8 + 1);
        fa_load(StepTag<2>{}, cb * 16 + wi * 8 + 2);
#pragma unroll
        for (int g = 0; g < NPMAX / 4; g++) patch_store(g, raw0);
#pragma unroll
        for (int g = 0; g < NPMAX / 4; g++)
            if (4 * g < nslots)
                *(float4 *)((char *)(raw0 + raw_floats) + p_lds + g * 16) =
                    make_float4(second[4 * g], second[4 * g + 1], second[4 * g + 2], second[4 * g + 3]);
    } else {
        fa_load(StepTag<0>{}, cb * 16 + wi * 8);
        fa_load(StepTag<1>{}, cb * 16 + wi * 8 + 1);
        fa_load(StepTag<2>{}, cb * 16 + wi * 8 + 2);
#pragma unroll
        for (int g = 0; g < NPMAX / 4; g++) patch_store(g, raw0);
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < 4; b++) transform_read(b, raw0);
    transform_write(V0);
    __syncthreads();

    constexpr int PER = NPMAX / 4;
    float4 fb_next[2];
    fb_next[0] = *(const float4 *)(V0 + b_frag);
    fb_next[1] = *(const float4 *)(V0 + b_frag + 4);
    for (int it = 0; it < nch; ++it) {
        const int chunk = cb + it;
        // double-buffered: V of this chunk, raw patch and V of the next one, raw patch of the one after (into the buffer
        // this chunk's patch left when it was transformed)
        const float *const Vc = V0 + (DB ? (it & 1) * VSZ : 0);
        float *const Vn = V0 + (DB ? ((it + 1) & 1) * VSZ : 0);
        const float *const rawn = raw0 + (DB ? ((it + 1) & 1) * raw_floats : 0);
        float *const raww = raw0 + (DB ? (it & 1) * raw_floats : 0);
        const int ahead = DB ? 2 : 1;
        const bool more = it + 1 < nch, fetch = it + ahead < nch;
        static_for<0, 8>([&](auto xtag) {
            constexpr int xl = decltype(xtag)::value;
            const float4 fb0 = fb_next[0], fb1 = fb_next[1];
            const float4 fa0 = fa_ring[xl % 4][0], fa1 = fa_ring[xl % 4][1];
            static_for<0, 8>([&](auto stag) {
                constexpr int ks = decltype(stag)::value;
                // side work of this step, pinned to it: left to itself the scheduler sinks every load to its first use
                if constexpr (ks == 0) {
                    // the filter fragments three positions ahead (into the slot of the position before this one)
                    fa_load(StepTag<(xl + 3) % 4>{}, (xl + 3 < 8 ? chunk * 16 : (chunk + 1) * 16 - 8) + wi * 8 + xl + 3);
                }
                if constexpr (ks == 1 && xl < 7) {   // this lane's tile at the next position
                    fb_next[0] = *(const float4 *)(Vc + b_frag + (xl + 1) * TT * LDP);
                    fb_next[1] = *(const float4 *)(Vc + b_frag + (xl + 1) * TT * LDP + 4);
                }
                // the patch `ahead` chunks on: loads during positions 0..3, LDS stores during 4..7
                if constexpr (xl < 4 && ks >= 2 && ks < 2 + PER) {
                    if (fetch) patch_load(xl * PER + ks - 2, chunk + ahead);
                }
                if constexpr (xl >= 4 && ks == 2) {
                    if (fetch) patch_store(xl - 4, raww);
                }
                if constexpr (DB && ks == 6) {       // the next chunk's transform: a column per position, then the products
                    if (more) {
                        if constexpr (xl < 4) transform_read(xl, rawn);
                        if constexpr (xl == 4) transform_write(Vn);
                    }
                }
                const float4 av = ks < 4 ? fa0 : fa1, bv = ks < 4 ? fb0 : fb1;
                const float a = ks % 4 == 0 ? av.x : ks % 4 == 1 ? av.y : ks % 4 == 2 ? av.z : av.w;
                const float b = ks % 4 == 0 ? bv.x : ks % 4 == 1 ? bv.y : ks % 4 == 2 ? bv.z : bv.w;
                acc[xl] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[xl], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        __syncthreads();              // every wavefront is done with V of this chunk; the next patch is in place
        if constexpr (!DB) {
            if (more) {
#pragma unroll
                for (int b = 0; b < 4; b++) transform_read(b, raw0);
                transform_write(V0);
            }
            __syncthreads();
        }
        fb_next[0] = *(const float4 *)(Vn + b_frag);
        fb_next[1] = *(const float4 *)(Vn + b_frag + 4);
    }

    // ---- inverse transform.  This wavefront's rows of the 4x4 grid are i = 2 wi, 2 wi + 1; acc[4 il + j] = M[i][j].
    // At = [1 1 1 0; 0 1 -1 -1]:  z[i][0] = m0 + m1 + m2, z[i][1] = m1 - m2 - m3, then the same over i.
    float *const xchg = lds;          // [wavefront pair][accumulator row][lane][4]: the main loop's LDS is free now
    float *outp = p.out + (size_t)split * p.out_elems;
    const bool add_bias = p.bias != nullptr && p.splits == 1;
    float part[16][4];                // per accumulator row v: this wavefront's share of y[a][b], index 2 a + b
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const float za0 = (acc[0][v] + acc[1][v]) + acc[2][v], za1 = (acc[1][v] - acc[2][v]) - acc[3][v];
        const float zb0 = (acc[4][v] + acc[5][v]) + acc[6][v], zb1 = (acc[5][v] - acc[6][v]) - acc[7][v];
        if (wi == 0) {                // rows 0, 1: y[0] += z0 + z1, y[1] += z1
            part[v][0] = za0 + zb0; part[v][1] = za1 + zb1; part[v][2] = zb0; part[v][3] = zb1;
        } else {                      // rows 2, 3: y[0] += z2, y[1] += -z2 - z3
            part[v][0] = za0; part[v][1] = za1; part[v][2] = -za0 - zb0; part[v][3] = -za1 - zb1;
        }
    }
    if (wi == 1) {   // a lane's four shares of one accumulator row are one 128-bit store
#pragma unroll
        for (int v = 0; v < 16; v++)
            *(float4 *)(xchg + (((w >> 1) * 16 + v) * 64 + lane) * 4) = make_float4(part[v][0], part[v][1], part[v][2], part[v][3]);
    }
    __syncthreads();
    if (wi == 1) return;
    {
        const int tau = th * 32 + l32, img = tau / tpi, tl = tau - img * tpi, r2 = tl / tcn, c2 = tl - r2 * tcn;
        const int n = n_first + img;
        if (n >= p.N) return;
        float *base = outp + ((size_t)n * p.Mout * p.OH + (oh0 + 2 * r2)) * p.OW + 2 * c2;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = m0 + wk * 32 + acc_row(v, lane);
            if (m >= p.Mout) continue;
            const float bias = add_bias ? p.bias[m] : 0.0f;
            const float4 other = *(const float4 *)(xchg + (((w >> 1) * 16 + v) * 64 + lane) * 4);
            float y[4] = {part[v][0] + other.x, part[v][1] + other.y, part[v][2] + other.z, part[v][3] + other.w};
            if (add_bias) {
#pragma unroll
                for (int q = 0; q < 4; q++) y[q] += bias;
            }
            float *o = base + (size_t)m * OHW;
            *(float2 *)o = make_float2(y[0], y[1]);
            *(float2 *)(o + p.OW) = make_float2(y[2], y[3]);
        }
    }
}

// The transformed filter of the Winograd kernel: U[((chunk*16 + xi)*Mp + m)*16 + j] = (G g Gt)[xi] for row m and
// channel chunk*16 + j, where g is the filter as the kernel applies it to the patch: g[r][s] multiplies patch offset
// (r, s), i.e. the stored taps read backwards when the operation is a true convolution (`flip`).  Staged like
// pack_tile (16 rows of one chunk); G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1].
template <bool kBwd>
__device__ __forceinline__ void wino_pack_tile(int M, int Cred, int Mp, size_t sm, size_t sc, int flip, const float *w, float *wp,
                                               int chunk, int m0, float *stage)
{
    constexpr int PITCH = kBwd ? 148 : 145;
    float v[9];
#pragma unroll
    for (int i = 0; i < 9; i++) {
        const int f = i * 256 + threadIdx.x;
        const int run = f / 144, r = f - run * 144;
        bool ok;
        size_t src;
        if (!kBwd) {
            ok = m0 + run < M && chunk * 16 + r / 9 < Cred;
            src = (size_t)(m0 + run) * sm + (size_t)chunk * 16 * sc + r;
        } else {
            ok = chunk * 16 + run < Cred && m0 + r / 9 < M;
            src = (size_t)(chunk * 16 + run) * sc + (size_t)m0 * sm + r;
        }
        v[i] = ok ? w[src] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 9; i++) {
        const int f = i * 256 + threadIdx.x;
        stage[(f / 144) * PITCH + f % 144] = v[i];
    }
    __syncthreads();
    // one (row, channel) pair per thread: 16 x 16 pairs, sixteen values each
    {
        const int j = threadIdx.x & 15, ml = threadIdx.x >> 4;
        const float *s = !kBwd ? stage + ml * PITCH + j * 9 : stage + j * PITCH + ml * 9;
        float g[3][3];
#pragma unroll
        for (int r = 0; r < 3; r++)
#pragma unroll
            for (int c = 0; c < 3; c++) g[r][c] = flip ? s[(2 - r) * 3 + (2 - c)] : s[r * 3 + c];
        float h[4][3];   // G g
#pragma unroll
        for (int c = 0; c < 3; c++) {
            h[0][c] = g[0][c];
            h[1][c] = ((g[0][c] + g[1][c]) + g[2][c]) * 0.5f;
            h[2][c] = ((g[0][c] - g[1][c]) + g[2][c]) * 0.5f;
            h[3][c] = g[2][c];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float u0 = h[r][0], u1 = ((h[r][0] + h[r][1]) + h[r][2]) * 0.5f, u2 = ((h[r][0] - h[r][1]) + h[r][2]) * 0.5f,
                        u3 = h[r][2];
            float *dst = wp + (((size_t)chunk * 16 + r * 4) * Mp + m0 + ml) * 16 + j;
            dst[0] = u0;
            dst[(size_t)Mp * 16] = u1;
            dst[(size_t)2 * Mp * 16] = u2;
            dst[(size_t)3 * Mp * 16] = u3;
        }
    }
}

// Packed filter of the patch kernel: wp[((chunk*9 + tap)*Mp + m)*16 + j] = w[m*sm + (chunk*16+j)*sc + tap]
// (zero where m >= M or the channel is past the end).  Forward: m = output channel k (sm = C*9,
// sc = 9); backward-data: m = input channel c (sm = 9, sc = C*9), reduction over k.
// A block transposes 16 rows of one chunk through LDS.  Its source is 16 contiguous runs of 144
// floats (forward: one per row, its 16 channels x 9 taps; backward: one per reduction channel,
// its 16 rows x 9 taps), copied to LDS as they lie -- all nine loads of a thread in flight at
// once; the scattered side of the transposition is the LDS read, whose strides spread the lanes
// over the banks.
template <bool kBwd>
__device__ __forceinline__ void pack_tile(int M, int Cred, int Mp, size_t sm, size_t sc, const float *w, float *wp,
                                          int chunk, int m0, float *stage)
{
    constexpr int PITCH = kBwd ? 148 : 145;  // floats between runs in LDS
    float v[9];
#pragma unroll
    for (int i = 0; i < 9; i++) {
        const int f = i * 256 + threadIdx.x;
        const int run = f / 144, r = f - run * 144;
        bool ok;
        size_t src;
        if (!kBwd) {  // run = row m0 + run, r = (channel, tap)
            ok = m0 + run < M && chunk * 16 + r / 9 < Cred;
            src = (size_t)(m0 + run) * sm + (size_t)chunk * 16 * sc + r;
        } else {      // run = reduction channel chunk*16 + run, r = (row, tap)
            ok = chunk * 16 + run < Cred && m0 + r / 9 < M;
            src = (size_t)(chunk * 16 + run) * sc + (size_t)m0 * sm + r;
        }
        v[i] = ok ? w[src] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 9; i++) {
        const int f = i * 256 + threadIdx.x;
        stage[(f / 144) * PITCH + f % 144] = v[i];
    }
    __syncthreads();
    // one float4 (four channels of one row and tap) per thread and pass
    for (int o = threadIdx.x; o < 9 * 16 * 4; o += 256) {
        const int j4 = o & 3, ml = (o >> 2) & 15, tap = o >> 6;
        float4 q;
        if (!kBwd) {
            const float *s = stage + ml * PITCH + (j4 * 4) * 9 + tap;
            q = make_float4(s[0], s[9], s[18], s[27]);
        } else {
            const float *s = stage + (j4 * 4) * PITCH + ml * 9 + tap;
            q = make_float4(s[0], s[PITCH], s[2 * PITCH], s[3 * PITCH]);
        }
        *(float4 *)&wp[(((size_t)chunk * 9 + tap) * Mp + m0 + ml) * 16 + j4 * 4] = q;
    }
}

template <bool kBwd>
__global__ __launch_bounds__(256) void pack_patch_k(int M, int Cred, int Mp, size_t sm, size_t sc, int wino, int flip,
                                                     const float *w, float *wp)
{
    __shared__ float stage[16 * 148];
    if (wino) wino_pack_tile<kBwd>(M, Cred, Mp, sm, sc, flip, w, wp, blockIdx.y, blockIdx.x * 16, stage);
    else pack_tile<kBwd>(M, Cred, Mp, sm, sc, w, wp, blockIdx.y, blockIdx.x * 16, stage);
}

// The filters of many layers in one launch (a training step packs each filter twice, once per
// direction, and most of those launches are far too small to fill the chip on their own).
constexpr int kPackJobs = 32;
struct PackJob {
    const float *w;
    float *wp;
    int M, Cred, Mp, bwd;
    int wino, flip;                  // wino: the Winograd kernel's transformed filter (16 positions per chunk instead of 9 taps)
    unsigned sm, sc;
    unsigned first_block, mblocks;   // blocks [first_block, next job's first_block): (chunk, row block) pairs
};
struct PackBatch {
    PackJob job[kPackJobs];
    int njobs;
};

__global__ __launch_bounds__(256) void pack_batch_k(PackBatch b)
{
    __shared__ float stage[16 * 148];
    int j = 0;
    while (j + 1 < b.njobs && blockIdx.x >= b.job[j + 1].first_block) j++;
    const PackJob &q = b.job[j];
    const unsigned local = blockIdx.x - q.first_block;
    const int chunk = (int)(local / q.mblocks), m0 = (int)(local % q.mblocks) * 16;
    if (q.wino) {
        if (q.bwd) wino_pack_tile<true>(q.M, q.Cred, q.Mp, q.sm, q.sc, q.flip, q.w, q.wp, chunk, m0, stage);
        else wino_pack_tile<false>(q.M, q.Cred, q.Mp, q.sm, q.sc, q.flip, q.w, q.wp, chunk, m0, stage);
    } else if (q.bwd) pack_tile<true>(q.M, q.Cred, q.Mp, q.sm, q.sc, q.w, q.wp, chunk, m0, stage);
    else pack_tile<false>(q.M, q.Cred, q.Mp, q.sm, q.sc, q.w, q.wp, chunk, m0, stage);
}

// ------------------------------------------------------------------------------------ backward-filter

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

// TPT = number of column groups of a tile that may belong to different taps (BN / gcd(BN, Cp)):
// the input displacement and the bounds test are per group, not per element.
template <class T, int TPT>
__global__ __launch_bounds__(T::THREADS, T::THREADS / 128) void conv_wgrad_k(FilterGrad p)
{
    constexpr int BM = T::BM, BN = T::BN, LDA = T::LDA, LDB = T::LDB;
    static_assert(T::THREADS == 256, "lanes run along 16 pixels, 16 rows per pass");
    constexpr int NA = BM / 16, NB = BN / 16;  // scalar loads per thread
    constexpr int GSZ = NB / TPT;              // loads per tap group
    static_assert(GSZ * TPT == NB, "TPT must divide the loads per thread");
    __shared__ float As[2][BK * LDA];
    __shared__ float Bs[2][BK * LDB];

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
    const int wm = w / T::WN, wn = w % T::WN;
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

    v16f acc[T::MI][T::NI];
    zero_acc(acc);
    load(slab_begin);
    store(0);
    __syncthreads();
    int cur = 0;
    for (int slab = slab_begin; slab < slab_end - 1; ++slab) {
        load(slab + 1);
        mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * (BM / T::WM), wn * (BN / T::WN), acc, lane);
        store(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    mma_slab<BK, LDA, LDB>(As[cur], Bs[cur], wm * (BM / T::WM), wn * (BN / T::WN), acc, lane);

    float *outp = p.out + (size_t)split * p.out_elems;
#pragma unroll
    for (int j = 0; j < T::NI; j++) {
        const int col = n0 + wn * (BN / T::WN) + j * 32 + (lane & 31);
        if (col >= p.ncols) continue;
#pragma unroll
        for (int i = 0; i < T::MI; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * (BM / T::WM) + i * 32 + acc_row(v, lane);
                if (m < p.K) outp[(size_t)m * p.ncols + col] = acc[i][j][v];
            }
    }
}

// dw[k][c][tap] = sum_s partial[s][k][tap*Cp + c], summed in a fixed order (reproducible).
// Block (k, chunk of `ch` channels): 64 element lanes x 4 split lanes.  Wavefront sl folds the
// splits s = sl, sl+4, ... of every element with four independent chains (the split count reaches
// the hundreds for the wide early layers, one dependent chain per element would be latency
// bound); the four wavefront sums are then added in order, and the chunk is written out
// contiguously in [c][tap] order.
__global__ __launch_bounds__(256) void wgrad_reduce_k(int K, int C, int Cp, int taps, int ch, int splits,
                                                       size_t split_stride, const float *partial, float *dw)
{
    extern __shared__ float lds[];  // part[4][ch*taps] then stage[ch*taps]
    const int k = blockIdx.x, c0 = blockIdx.y * ch;
    const int nc = min(ch, C - c0);
    const int nelem = nc * taps, cap = ch * taps;
    float *part = lds, *stage = lds + 4 * cap;
    const int el = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const float *src = partial + (size_t)k * taps * Cp + c0;
    for (int i = el; i < nelem; i += 64) {
        const int t = i / nc, c = i - t * nc;
        const float *q = src + (size_t)t * Cp + c;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        int sp = sl;
        for (; sp + 12 < splits; sp += 16) {
            a0 += q[(size_t)sp * split_stride];
            a1 += q[(size_t)(sp + 4) * split_stride];
            a2 += q[(size_t)(sp + 8) * split_stride];
            a3 += q[(size_t)(sp + 12) * split_stride];
        }
        for (; sp < splits; sp += 4) a0 += q[(size_t)sp * split_stride];
        part[sl * cap + i] = (a0 + a1) + (a2 + a3);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nelem; i += 256) {
        const int t = i / nc, c = i - t * nc;
        stage[c * taps + t] = (part[i] + part[cap + i]) + (part[2 * cap + i] + part[3 * cap + i]);
    }
    __syncthreads();
    float *dst = dw + ((size_t)k * C + c0) * taps;
    for (int i = threadIdx.x; i < nelem; i += 256) dst[i] = stage[i];
}

// out[i] = sum over s of partial[s * stride + i], in a fixed order: split lane sl of a block folds
// the splits s = sl, sl + SL, ... (four independent chains, then ((a0+a1)+(a2+a3))), and the SL
// lane sums are added in lane order.  256 threads = (256 / SL) float4 columns x SL split lanes; SL
// is chosen by the host so that small outputs with hundreds of splits still fill the machine.
template <int SL>
__global__ __launch_bounds__(256) void split_sum_k(size_t n4, int splits, size_t stride4, const float4 *partial,
                                                    float4 *out)
{
    constexpr int EL = 256 / SL;
    __shared__ float4 part[SL][EL];
    const int el = threadIdx.x % EL, sl = threadIdx.x / EL;
    const size_t i = (size_t)blockIdx.x * EL + el;
    float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0, a2 = a0, a3 = a0;
    if (i < n4) {
        const float4 *q = partial + i;
        int sp = sl;
        for (; sp + 3 * SL < splits; sp += 4 * SL) {
            const float4 v0 = q[(size_t)sp * stride4], v1 = q[(size_t)(sp + SL) * stride4];
            const float4 v2 = q[(size_t)(sp + 2 * SL) * stride4], v3 = q[(size_t)(sp + 3 * SL) * stride4];
            a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
            a1.x += v1.x; a1.y += v1.y; a1.z += v1.z; a1.w += v1.w;
            a2.x += v2.x; a2.y += v2.y; a2.z += v2.z; a2.w += v2.w;
            a3.x += v3.x; a3.y += v3.y; a3.z += v3.z; a3.w += v3.w;
        }
        for (; sp < splits; sp += SL) {
            const float4 v0 = q[(size_t)sp * stride4];
            a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
        }
    }
    part[sl][el] = make_float4((a0.x + a1.x) + (a2.x + a3.x), (a0.y + a1.y) + (a2.y + a3.y),
                               (a0.z + a1.z) + (a2.z + a3.z), (a0.w + a1.w) + (a2.w + a3.w));
    __syncthreads();
    if (sl == 0 && i < n4) {
        float4 r = part[0][el];
#pragma unroll
        for (int k = 1; k < SL; k++) {
            const float4 v = part[k][el];
            r.x += v.x; r.y += v.y; r.z += v.z; r.w += v.w;
        }
        out[i] = r;
    }
}

// ------------------------------------------------------------------------------------ backward-filter, 3x3 patch
//
// Filter gradient of 3x3, unit-stride, pad-1 convolutions:
//   dw[k][c][2-r][2-s] = sum over (n, p, q) of dy[n][k][p][q] * x[n][c][p-1+r][q-1+s].
// The reduction runs over pixels.  A block owns BM output channels x BC input channels x all nine
// taps (BM x BC = 128 x 32, 64 x 64, or 160 x 32 for layers of 160 channels, which the other two would pad by
// a fifth and more) and walks the pixels in chunks of 64.  Per chunk it stages dy[BM][64] and ONE zero-haloed
// patch of x for its BC channels in LDS; the nine taps read that patch at nine offsets, so x is
// fetched once, not nine times.  The twelve wavefronts are (32 rows of k) x (32 channels) x
// (tap row r): a wavefront keeps the three taps s = 0..2 of its tap row in three 32x32
// accumulators.  A lane's operands for a 16-pixel slab are pixels kh*8 .. kh*8+7 of the slab
// (kh = lane / 32): two 128-bit reads of dy, and for x a window that serves all three taps by
// register selection.
//
// Geometry of a 64-pixel chunk (kGeo):
//   0  rows of 8, 16, 32 or 64 pixels: G = 64/W full rows of one image.  Patch rows have pitch W+8
//      with pixel q at column q+4, so interior quads are 16-byte aligned; a lane's window is two
//      aligned quads plus the two edge columns.  The halo rows above and below are fetched (or
//      masked at the image border); the halo columns are cleared once and never written.
//   1  4x4 images: four whole images.  Same column layout (pitch 12); a lane's 8 pixels are two
//      rows, each one aligned quad plus two edge columns.  All halo cells stay zero.
//   2  2x2 images: sixteen whole images, each a 4x4 cell block with the image in the middle; a
//      lane's 8 pixels are two images, and one aligned quad per (image, row) holds every column
//      the three taps need.

struct WgradPatch {
    const float *dy;  // [N, K, H, W]
    const float *x;   // [N, C, H, W]
    float *out;       // dw [K][C][3][3], or `splits` partial copies of it `split_stride` floats apart
    size_t split_stride;
    int N, C, K, H, W;
    int G, bands;         // geometry 0: output rows per chunk (G*W = 64), chunks per image; else 1
    int imgs;             // images per chunk (1, 4 or 16)
    int ppitch, cstride;  // patch row pitch; floats per channel (128-bit reads by 32 channels hit every bank once)
    int quads_row;        // W / 4 (geometry 0)
    int mtiles, ctiles, chunks_total, chunks_per_split, splits;
    size_t dy_bytes, x_bytes;
};

template <int WM, int WC, int kGeo>
__device__ __forceinline__ void conv_wgrad_patch_body(const WgradPatch &p, const unsigned block_id)
{
    constexpr int BM = 32 * WM, BC = 32 * WC, THREADS = 64 * 3 * WM * WC, NPIX = 64, APITCH = NPIX + 4;
    constexpr int NAQ = (BM * NPIX / 4 + THREADS - 1) / THREADS;  // float4 slots of dy per thread
    // float4 slots of x per thread: geometry 0 up to 32*4*8 (W = 32) or 32*3*16 (W = 64) quads per 32
    // channels; geometries 1, 2 have 16 quads per channel
    constexpr int NBQ = kGeo == 0 ? (WC == 1 ? 2 : 3) : (BC * 16 + THREADS - 1) / THREADS;
    static_assert(WM * WC == 4 || WM * WC == 5, "twelve or fifteen wavefronts: 4 or 5 (row, channel) groups x 3 tap rows");
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int bsize = BC * p.cstride;
    float *const A0 = lds;                     // [2][BM * APITCH]
    float *const B0 = lds + 2 * BM * APITCH;   // [2][bsize]
    float *const dummy = B0 + 2 * bsize;       // 4 floats absorbing the stores of unused slots

    unsigned L;
    const unsigned tiles = (unsigned)(p.mtiles * p.ctiles);
    if (!xcd_remap(block_id, tiles * (unsigned)p.splits, &L)) return;
    const int split = (int)(L / tiles);
    const unsigned tile = L - (unsigned)split * tiles;
    const int mt = (int)(tile % (unsigned)p.mtiles), ct = (int)(tile / (unsigned)p.mtiles);
    const int k0 = mt * BM, c0 = ct * BC;
    const int cb = split * p.chunks_per_split;
    const int ce = min(cb + p.chunks_per_split, p.chunks_total);

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int kh = lane >> 5, l32 = lane & 31;
    const int dr = w % 3, grp = w / 3;
    const int wm = grp / WC, wc = grp % WC;
    const int HW = p.H * p.W;

    const __amdgpu_buffer_rsrc_t rdy = make_rsrc(p.dy, p.dy_bytes);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x, p.x_bytes);

    // ---- load slots.  dy: quad `quad` of row `row` is pixels 4*quad .. 4*quad+3 of the chunk, which
    // lie in image quad / qpi of the chunk (qpi = quads of one image inside a chunk).
    unsigned a_voff[NAQ];
    int a_lds[NAQ];
    const int qpi = kGeo == 0 ? 16 : HW / 4;
#pragma unroll
    for (int i = 0; i < NAQ; i++) {
        const int a = i * THREADS + tid;
        const int row = a / 16, quad = a % 16;
        const int j = quad / qpi, wq = quad - j * qpi;
        const bool ok = a < BM * 16 && k0 + row < p.K;
        a_voff[i] = ok ? (unsigned)((j * p.K + k0 + row) * HW + wq * 4) * 4u : kOobOffset;
        a_lds[i] = a < BM * 16 ? row * APITCH + quad * 4 : -1;
    }
    unsigned b_voff[NBQ];
    int b_lds[NBQ], b_edge[NBQ];  // b_edge (geometry 0): 1 = top halo row, 2 = bottom halo row
#pragma unroll
    for (int i = 0; i < NBQ; i++) {
        const int b = i * THREADS + tid;
        if (kGeo == 0) {
            const int quads_ch = (p.G + 2) * p.quads_row;
            const int c = b / quads_ch, rem = b - c * quads_ch;
            const int pr = rem / p.quads_row, quad = rem - pr * p.quads_row;
            const bool ok = c < BC && c0 + c < p.C;
            // row p0 - 1 + pr of channel c0 + c; p0 and the image are added per chunk
            b_voff[i] = ok ? (unsigned)(((c0 + c) * p.H + pr) * p.W + quad * 4) * 4u : kOobOffset;
            b_lds[i] = c < BC ? c * p.cstride + pr * p.ppitch + 4 + quad * 4 : -1;
            b_edge[i] = pr == 0 ? 1 : (pr == p.G + 1 ? 2 : 0);
        } else if (kGeo == 1) {
            const int c = b / 16, j = (b / 4) % 4, row = b % 4;  // image j of the chunk, image row `row`
            const bool ok = c < BC && c0 + c < p.C;
            b_voff[i] = ok ? (unsigned)((j * p.C + c0 + c) * 16 + row * 4) * 4u : kOobOffset;
            b_lds[i] = c < BC ? c * p.cstride + j * 72 + (row + 1) * 12 + 4 : -1;
            b_edge[i] = 0;
        } else {
            const int c = b / 16, j = b % 16;  // the whole 2x2 image j is one quad
            const bool ok = c < BC && c0 + c < p.C;
            b_voff[i] = ok ? (unsigned)((j * p.C + c0 + c) * 4) * 4u : kOobOffset;
            b_lds[i] = c < BC ? c * p.cstride + j * 16 + 5 : -1;  // cell (1,1) of the 4x4 block
            b_edge[i] = 0;
        }
    }
    float4 areg[NAQ], breg[NBQ];
    // position of the chunk being FETCHED: first image and, for geometry 0, the band of rows
    int n_img = kGeo == 0 ? cb / p.bands : cb * p.imgs, band = kGeo == 0 ? cb - n_img * p.bands : 0;
    auto fetch = [&]() {
        const int p0 = band * p.G;
        const unsigned a_soff = (unsigned)(n_img * p.K * HW + p0 * p.W) * 4u;
#pragma unroll
        for (int i = 0; i < NAQ; i++) areg[i] = buffer_load_f32x4(rdy, a_voff[i], a_soff);
        if (kGeo == 0) {
            // x row p0 - 1 + pr.  Offsets handed to a buffer load must not go negative: the "- 1" row
            // is taken off the wave-uniform part, except for the very first chunk of the tensor, where
            // it is taken off the per-lane part (whose top halo row, the only one it could underflow,
            // is masked)
            const int kill = (band == 0 ? 1 : 0) | (band == p.bands - 1 ? 2 : 0);
            const bool first = n_img == 0 && band == 0;
            const unsigned roww = (unsigned)p.W * 4u;
            const unsigned b_soff = (unsigned)(n_img * p.C * HW + p0 * p.W) * 4u - (first ? 0u : roww);
#pragma unroll
            for (int i = 0; i < NBQ; i++) {
                const bool dead = (b_edge[i] & kill) != 0 || b_voff[i] == kOobOffset;
                breg[i] = buffer_load_f32x4(rx, dead ? kOobOffset : b_voff[i] - (first ? roww : 0u), b_soff);
            }
            if (++band == p.bands) {
                band = 0;
                ++n_img;
            }
        } else {
            const unsigned b_soff = (unsigned)(n_img * p.C * HW) * 4u;
#pragma unroll
            for (int i = 0; i < NBQ; i++) breg[i] = buffer_load_f32x4(rx, b_voff[i], b_soff);
            n_img += p.imgs;
        }
    };
    auto stash = [&](int buf) {
        float *A = A0 + buf * (BM * APITCH), *B = B0 + buf * bsize;
#pragma unroll
        for (int i = 0; i < NAQ; i++) *(float4 *)(a_lds[i] >= 0 ? A + a_lds[i] : dummy) = areg[i];
#pragma unroll
        for (int i = 0; i < NBQ; i++) {
            if (kGeo != 2) {
                *(float4 *)(b_lds[i] >= 0 ? B + b_lds[i] : dummy) = breg[i];
            } else {
                float *q = b_lds[i] >= 0 ? B + b_lds[i] : dummy;  // rows 1 and 2 of the cell block, columns 1..2
                const int down = b_lds[i] >= 0 ? 4 : 0;
                q[0] = breg[i].x;
                q[1] = breg[i].y;
                q[down] = breg[i].z;
                q[down + 1] = breg[i].w;
            }
        }
    };

    // ---- fragment addresses
    const int a_frag = (wm * 32 + l32) * APITCH + kh * 8;
    int b_frag[4];  // float4 index inside a patch buffer, per slab
    const int chan = (wc * 32 + l32) * p.cstride;
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (kGeo == 0) {
            // slab s covers the 8-pixel runs 2s (kh = 0) and 2s+1 (kh = 1) of the chunk
            const int runs_row = p.W / 8;
            const int u = 2 * s + kh, rho = u / runs_row, q0 = (u - rho * runs_row) * 8;
            b_frag[s] = (chan + (rho + dr) * p.ppitch + q0) / 4 + 1;  // quad of pixel q0
        } else if (kGeo == 1) {
            b_frag[s] = (chan + s * 72 + (2 * kh + dr) * 12) / 4 + 1;  // image s, image rows 2kh and 2kh+1
        } else {
            b_frag[s] = (chan + (4 * s + 2 * kh) * 16 + dr * 4) / 4;   // images 4s+2kh and 4s+2kh+1
        }
    }

    // halo cells are never written again: clear both patch buffers once
    for (int i = tid; i < 2 * bsize; i += THREADS) B0[i] = 0.0f;
    __syncthreads();

    v16f acc[3];
#pragma unroll
    for (int t = 0; t < 3; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;

    fetch();
    stash(0);
    __syncthreads();
    int cur = 0;
    typedef __attribute__((address_space(3))) float lds_float_t;
    // Fetching runs one chunk ahead and also past the end of this block's range: those loads are
    // range-checked and their data lands in the LDS buffer that is not read again.
    // The fragments of a step are read one step ahead (the first step's after the barrier that releases the chunk), so
    // that their LDS latency passes under the previous step's matrix instructions - with twelve wavefronts; fifteen have
    // 128 registers each and no room for a second set.
    constexpr bool AHEAD = WM * WC == 4;
    struct Frag {
        float4 a_lo, a_hi, q[4];
        float e[4];
    };
    auto read_frag = [&](int buf, int s_) {
        Frag f;
        const float *A = A0 + buf * (BM * APITCH) + a_frag;
        // float4 indexing keeps the 16-byte alignment of the patch reads visible to the compiler
        const float4 *bq = (const float4 *)B0 + buf * (bsize / 4) + b_frag[s_];
        // The edge-column reads are volatile so that the compiler does not fuse a whole window
        // into one run starting at the unaligned edge (it would then read it in 2-dword pieces).
        const volatile lds_float_t *be = (const volatile lds_float_t *)bq;
        f.a_lo = *(const float4 *)(A + s_ * 16);
        f.a_hi = *(const float4 *)(A + s_ * 16 + 4);
        if constexpr (kGeo == 0) {
            f.q[0] = bq[0]; f.q[1] = bq[1];
            f.e[0] = be[-1]; f.e[1] = be[8];
        } else if constexpr (kGeo == 1) {
            f.q[0] = bq[0]; f.q[1] = bq[3];   // the next patch row is 12 floats on
            f.e[0] = be[-1]; f.e[1] = be[4]; f.e[2] = be[11]; f.e[3] = be[16];
        } else {
            // (image, row) quads: image 0 rows 0, 1 then image 1 rows 0, 1
            f.q[0] = bq[0]; f.q[1] = bq[1]; f.q[2] = bq[4]; f.q[3] = bq[5];
        }
        return f;
    };
    Frag nxt;
    if constexpr (AHEAD) nxt = read_frag(0, 0);
    for (int chunk = cb; chunk < ce; ++chunk) {
        static_for<0, 4>([&](auto stag) {
            constexpr int s = decltype(stag)::value;
            if constexpr (s == 0) fetch();
            Frag f;
            if constexpr (AHEAD) {
                f = nxt;
                if constexpr (s < 3) {
                    nxt = read_frag(cur, s + 1);
                    __builtin_amdgcn_sched_barrier(0);   // issued here, not where they are first used
                }
            } else {
                f = read_frag(cur, s);
            }
            const float a8[8] = {f.a_lo.x, f.a_lo.y, f.a_lo.z, f.a_lo.w, f.a_hi.x, f.a_hi.y, f.a_hi.z, f.a_hi.w};
            if constexpr (kGeo == 0) {
                const float4 b_lo = f.q[0], b_hi = f.q[1];
                const float win[10] = {f.e[0], b_lo.x, b_lo.y, b_lo.z, b_lo.w, b_hi.x, b_hi.y, b_hi.z, b_hi.w, f.e[1]};
#pragma unroll
                for (int ks = 0; ks < 8; ks++)
#pragma unroll
                    for (int ds = 0; ds < 3; ds++)
                        acc[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(a8[ks], win[ks + ds], acc[ds], 0, 0, 0);
            } else if constexpr (kGeo == 1) {
                const float4 r0 = f.q[0], r1 = f.q[1];
                const float w0[6] = {f.e[0], r0.x, r0.y, r0.z, r0.w, f.e[1]};
                const float w1[6] = {f.e[2], r1.x, r1.y, r1.z, r1.w, f.e[3]};
#pragma unroll
                for (int ks = 0; ks < 8; ks++)
#pragma unroll
                    for (int ds = 0; ds < 3; ds++)
                        acc[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(a8[ks], ks < 4 ? w0[ks + ds] : w1[ks - 4 + ds],
                                                                       acc[ds], 0, 0, 0);
            } else {
                // pixel (row, col) of tap column ds reads element col + ds of the quad of patch row row + dr
                const float4 q00 = f.q[0], q01 = f.q[1], q10 = f.q[2], q11 = f.q[3];
                const float win[4][4] = {{q00.x, q00.y, q00.z, q00.w}, {q01.x, q01.y, q01.z, q01.w},
                                         {q10.x, q10.y, q10.z, q10.w}, {q11.x, q11.y, q11.z, q11.w}};
#pragma unroll
                for (int ks = 0; ks < 8; ks++)
#pragma unroll
                    for (int ds = 0; ds < 3; ds++)
                        acc[ds] = __builtin_amdgcn_mfma_f32_32x32x2f32(a8[ks], win[ks / 2][(ks & 1) + ds], acc[ds], 0, 0, 0);
            }
            if constexpr (s == 3) stash(cur ^ 1);
        });
        __syncthreads();
        cur ^= 1;
        if constexpr (AHEAD) nxt = read_frag(cur, 0);   // (past the last chunk: the buffer the final, unused prefetch was stored to)
    }

    // Epilogue: the accumulators leave through LDS so that every output row -- the BC*9 values
    // [c][tap] of one k, contiguous in dw's own layout -- is written as one run.  One group of 32
    // rows (the wavefronts with the same wm) is staged per pass.  out = dw itself when there is one
    // split, else this split's partial copy (same layout, summed afterwards in split order).
    __syncthreads();  // all fragment reads of the last chunk are done: LDS is free
    constexpr int RP = BC * 9 + 1;  // staging row pitch (odd: the 4-row stride between lane halves spreads over banks)
    float *outp = p.out + (size_t)split * p.split_stride;
    const int ncv = min(BC, p.C - c0) * 9;  // valid floats of a staged row
    for (int g = 0; g < WM; g++) {
        if (wm == g) {
#pragma unroll
            for (int ds = 0; ds < 3; ds++) {
                const int t = (2 - dr) * 3 + (2 - ds);
#pragma unroll
                for (int v = 0; v < 16; v++) lds[acc_row(v, lane) * RP + (wc * 32 + l32) * 9 + t] = acc[ds][v];
            }
        }
        __syncthreads();
        for (int r = w; r < 32; r += 3 * WM * WC) {  // one wavefront per row
            const int k = k0 + g * 32 + r;
            if (k >= p.K) continue;
            float *dst = outp + ((size_t)k * p.C + c0) * 9;
            for (int j = lane; j < ncv; j += 64) dst[j] = lds[r * RP + j];
        }
        __syncthreads();
    }
}

template <int WM, int WC, int kGeo>
__global__ __launch_bounds__(64 * 3 * WM * WC, 1) void conv_wgrad_patch_k(WgradPatch p)
{
    conv_wgrad_patch_body<WM, WC, kGeo>(p, blockIdx.x);
}

// Backward-data and filter gradient of one layer in ONE launch: both read dy and nothing of each other.
// The first `grid_a` workgroups run the backward-data tiles, the rest the filter-gradient tiles; workgroups are
// dispatched in id order, so a compute unit that has finished its backward-data tile starts a filter-gradient
// tile at once instead of idling until the slowest tile of the launch is done and the next launch has ramped up.
// Launched with the filter gradient's 768 threads: the wavefronts a backward-data workgroup does not need end
// at once (a barrier waits for the surviving wavefronts only).
template <class T, int NPMAX, int WM, int WC, int kGeo>
__global__ __launch_bounds__(768, 1) void conv_bwd_pair_k(PatchConv a, WgradPatch b, unsigned grid_a)
{
    if (blockIdx.x < grid_a) {
        if (threadIdx.x >= (unsigned)T::THREADS) return;
        conv_patch_body<T, NPMAX, true>(a, blockIdx.x);
    } else {
        conv_wgrad_patch_body<WM, WC, kGeo>(b, blockIdx.x - grid_a);
    }
}

// ------------------------------------------------------------------------------------ helpers

// out[i] = sum_s partial[s][i], s ascending; plus bias[channel of i] when a bias is given
// (channel = (i / inner) % C for an [N, C, inner] output).
// kS > 0: exactly kS splits, all loads issued before the first add.
template <int kS>
__global__ __launch_bounds__(256) void splitk_reduce_k(size_t n4, int splits, const float4 *partial, float4 *out,
                                                        const float *bias, unsigned C, unsigned inner)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        if constexpr (kS > 0) {
            float4 v[kS];
#pragma unroll
            for (int s = 0; s < kS; s++) v[s] = partial[(size_t)s * n4 + i];
            acc = v[0];
#pragma unroll
            for (int s = 1; s < kS; s++) {
                acc.x += v[s].x;
                acc.y += v[s].y;
                acc.z += v[s].z;
                acc.w += v[s].w;
            }
        } else {
            // Rounds of four loads in flight (indices clamped to the last split, surplus values
            // dropped); the adds stay in ascending split order.
            const int last = splits - 1;
            for (int s = 0; s < splits; s += 4) {
                const float4 v0 = partial[(size_t)s * n4 + i];
                const float4 v1 = partial[(size_t)min(s + 1, last) * n4 + i];
                const float4 v2 = partial[(size_t)min(s + 2, last) * n4 + i];
                const float4 v3 = partial[(size_t)min(s + 3, last) * n4 + i];
                const bool h1 = s + 1 <= last, h2 = s + 2 <= last, h3 = s + 3 <= last;
                if (s == 0) acc = v0;   // not 0 + v0: the sum of negative zeros stays a negative zero
                else acc = make_float4(acc.x + v0.x, acc.y + v0.y, acc.z + v0.z, acc.w + v0.w);
                if (h1) acc = make_float4(acc.x + v1.x, acc.y + v1.y, acc.z + v1.z, acc.w + v1.w);
                if (h2) acc = make_float4(acc.x + v2.x, acc.y + v2.y, acc.z + v2.z, acc.w + v2.w);
                if (h3) acc = make_float4(acc.x + v3.x, acc.y + v3.y, acc.z + v3.z, acc.w + v3.w);
            }
        }
        if (bias) {
            const size_t e = i * 4;
            acc.x += bias[(e / inner) % C];
            acc.y += bias[((e + 1) / inner) % C];
            acc.z += bias[((e + 2) / inner) % C];
            acc.w += bias[((e + 3) / inner) % C];
        }
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

// DOPT_HIP_NO_TALL=1 keeps the 160-row tiles out (for A/B measurements); read once.
bool no_tall_tiles()
{
    static const bool off = std::getenv("DOPT_HIP_NO_TALL") != nullptr;
    return off;
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

int launch_splitk_reduce(size_t elems, int splits, const float *partial, float *out, const float *bias = nullptr,
                         unsigned C = 1, unsigned inner = 1)
{
    // float4 passes: the caller only splits when elems % 4 == 0, and the partial copies start on
    // 256-byte boundaries of the workspace; `out` comes from the pool or is checked by the caller
    const size_t n4 = elems / 4;
    size_t blocks = ceil_div(n4, (size_t)256);
    size_t cap = (size_t)num_cus() * 8;
    const dim3 grid((unsigned)(blocks > cap ? cap : (blocks < 1 ? 1 : blocks)));
    const float4 *p4 = (const float4 *)partial;
    float4 *o4 = (float4 *)out;
    switch (splits) {
    case 2: hipLaunchKernelGGL(splitk_reduce_k<2>, grid, dim3(256), 0, stream(), n4, splits, p4, o4, bias, C, inner); break;
    case 3: hipLaunchKernelGGL(splitk_reduce_k<3>, grid, dim3(256), 0, stream(), n4, splits, p4, o4, bias, C, inner); break;
    case 4: hipLaunchKernelGGL(splitk_reduce_k<4>, grid, dim3(256), 0, stream(), n4, splits, p4, o4, bias, C, inner); break;
    default: hipLaunchKernelGGL(splitk_reduce_k<0>, grid, dim3(256), 0, stream(), n4, splits, p4, o4, bias, C, inner); break;
    }
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

using GatherWide = Tile<64, 256, 1, 4>;     // few output channels, many pixels
using GatherSquare = Tile<128, 128, 2, 2>;  // enough tiles for two workgroups per CU
using GatherDeep = Tile<128, 128, 2, 4>;    // few tiles: 8 wavefronts per workgroup, one workgroup per CU
using GatherTall = Tile<160, 128, 1, 4>;    // 160 output channels (and 480, ...): 64- and 128-row tiles would multiply a fifth more rows than there are

unsigned div_magic(unsigned d) { return (unsigned)((((unsigned long long)1 << 32) / d) + 1); }

template <class T, int NPMAX>
int launch_patch(const PatchConv &pc, bool c_full, dim3 grid, size_t lds_bytes)
{
    // above 64 KB of dynamic LDS a kernel has to be told once
    static bool raised[2] = {false, false};
    if (!raised[c_full]) {
        const void *fn = c_full ? (const void *)conv_patch_k<T, NPMAX, true> : (const void *)conv_patch_k<T, NPMAX, false>;
        DOPT_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised[c_full] = true;
    }
    if (c_full) hipLaunchKernelGGL((conv_patch_k<T, NPMAX, true>), grid, dim3(T::THREADS), lds_bytes, stream(), pc);
    else hipLaunchKernelGGL((conv_patch_k<T, NPMAX, false>), grid, dim3(T::THREADS), lds_bytes, stream(), pc);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// 3x3 unit-stride layers whose pixel tiles are whole rows of one image or whole images.
// Returns DOPT_HIP_OK with *done = false when the layer does not fit this path.
// What the patch kernel needs to know about one convolution, without any pointer: which tile
// shape runs it and how its filter is packed.  `ok` is false when the generic kernel takes the shape.
struct PatchSetup {
    bool ok;
    PatchConv pc;
    int shape;            // 0 wide, 1 square, 2 deep, 3 tall, 4 Winograd (BM 128: 128 rows x 32 tiles of 2x2 pixels, BM 64: 64 rows x 64 tiles)
    int BM, BN, blocks_wanted, tiles;
    size_t lds_bytes, wp_elems;
};

template <bool kBwd>
PatchSetup patch_setup_as(const dopt_hip_conv_desc *d, size_t P, size_t Q, bool allow_tall, int wino = 0);   // wino: rows of a Winograd tile, 0 none

// DOPT_HIP_NO_WINO=1 keeps the Winograd kernel out (for A/B measurements); read once.
bool no_wino()
{
    static const bool off = std::getenv("DOPT_HIP_NO_WINO") != nullptr;
    return off;
}

// (a layer the 160-row tiles do not take - its pixel tile does not fit their patch - is tried with the other heights)
template <bool kBwd>
PatchSetup patch_setup(const dopt_hip_conv_desc *d, size_t P, size_t Q)
{
    if (!no_wino()) {
        // 128-row tiles first: measured faster than 64-row tiles on every layer that has both (they read the input once
        // per 128 rows and transform it once)
        const PatchSetup v = patch_setup_as<kBwd>(d, P, Q, false, 128);
        if (v.ok) return v;
        const PatchSetup v2 = patch_setup_as<kBwd>(d, P, Q, false, 64);
        if (v2.ok) return v2;
    }
    const PatchSetup u = patch_setup_as<kBwd>(d, P, Q, true);
    return u.ok ? u : patch_setup_as<kBwd>(d, P, Q, false);
}

template <bool kBwd>
PatchSetup patch_setup_as(const dopt_hip_conv_desc *d, size_t P, size_t Q, bool allow_tall, int wino)
{
    PatchSetup u{};
    if (d->R != 3 || d->S != 3 || d->strideH != 1 || d->strideW != 1 || d->padH > 2 || d->padW > 2) return u;
    PatchConv &pc = u.pc;
    pc.N = (int)d->N;
    if (!kBwd) {
        pc.Cin = (int)d->C; pc.IH = (int)d->H; pc.IW = (int)d->W;
        pc.Mout = (int)d->K; pc.OH = (int)P; pc.OW = (int)Q;
        pc.PT = (int)d->padH; pc.PL = (int)d->padW; pc.flip = 1;
    } else {
        pc.Cin = (int)d->K; pc.IH = (int)P; pc.IW = (int)Q;
        pc.Mout = (int)d->C; pc.OH = (int)d->H; pc.OW = (int)d->W;
        pc.PT = 2 - (int)d->padH; pc.PL = 2 - (int)d->padW; pc.flip = 0;
    }
    pc.ncols = pc.N * pc.OH * pc.OW;
    int npmax, threads;
    // 160-row tiles where they pad no more than both other heights (160 channels: 160 rows, not 192 or 256; 320 and 640
    // channels: two and four such tiles - on 8 x 8 images 640 channels are then exactly 256 tiles, one per compute unit
    // with no split of the reduction, where 128-row tiles gave 320 and a four-way split); 64-row tiles for up to 64 output
    // channels, and wherever 128-row tiles would pad more
    const int up64 = (pc.Mout + 63) / 64 * 64, up128 = (pc.Mout + 127) / 128 * 128, up160 = (pc.Mout + 159) / 160 * 160;
    // (only where they still give every compute unit a tile: 480 channels on 8 x 8 images are 192 such tiles, and ran slower)
    const long tall_tiles = (long)(up160 / 160) * ((pc.ncols + 127) / 128);
    if (wino) {
        // whole 16-channel chunks of a deep reduction, pad 1, 2 x 2 tiles
        if (d->padH != 1 || d->padW != 1 || pc.Cin % 16 != 0 || pc.Cin < 64 || pc.OH % 2 != 0 || pc.OW % 2 != 0 || pc.OH < 4 ||
            pc.OW < 4)
            return u;
        // whole tiles of rows, or 64-row tiles padded by no more than a fifth (160 rows as 192: still 1.9 times fewer
        // matrix instructions than the direct kernels execute)
        if (pc.Mout % wino != 0 && !(wino == 64 && pc.Mout > 64 && up64 * 5 <= pc.Mout * 6)) return u;
        // whole 128-row tiles of 32 tiles (128 pixels), or whole 64-row tiles of 64 tiles (256 pixels)
        u.shape = 4; u.BM = wino; u.BN = u.BM == 128 ? 128 : 256;
        u.blocks_wanted = num_cus(); npmax = 16; threads = 512;
    } else if (allow_tall && pc.Mout > 64 && up160 <= up64 && up160 <= up128 && tall_tiles >= num_cus() &&
        !no_tall_tiles()) {
        u.shape = 3; u.BM = 160; u.BN = 128; u.blocks_wanted = num_cus(); npmax = 16; threads = 256;
    } else if (pc.Mout <= 64 || up64 < up128) {
        u.shape = 0; u.BM = 64; u.BN = 256; u.blocks_wanted = 2 * num_cus(); npmax = 24; threads = 256;
    } else {
        u.BM = 128; u.BN = 128;
        const int t = ((pc.Mout + 127) / 128) * ((pc.ncols + 127) / 128);
        if (t >= 2 * num_cus()) { u.shape = 1; u.blocks_wanted = 2 * num_cus(); npmax = 16; threads = 256; }
        else { u.shape = 2; u.blocks_wanted = num_cus(); npmax = 16; threads = 512; }
    }
    const int BM = u.BM, BN = u.BN;
    // pixel tile = `rows` full rows of one image, or `nimg` whole images
    if (BN % pc.OW != 0) return u;
    const int tile_rows = BN / pc.OW;
    if (tile_rows <= pc.OH) {
        if (pc.OH % tile_rows != 0) return u;
        pc.nimg = 1; pc.rows = tile_rows;
    } else {
        if (tile_rows % pc.OH != 0) return u;
        pc.nimg = tile_rows / pc.OH; pc.rows = pc.OH;
    }
    pc.PR = pc.rows + 2; pc.PC = pc.OW + 2;
    pc.psz = pc.nimg * pc.PR * pc.PC;
    if ((size_t)pc.psz * 16 > (size_t)npmax * threads) return u;
    u.lds_bytes = (size_t)2 * (pc.psz + 1) * 20 * sizeof(float);
    if (wino) {
        if (pc.rows % 2 != 0) return u;   // a pixel tile is whole 2 x 2 tiles
        const size_t buffers = u.BM == 128 ? 2 : 1;   // 32 tiles: raw patch and V are double-buffered
        const size_t floats = buffers * ((size_t)(((pc.psz + 1) * 20 + 3) / 4 * 4) + (size_t)16 * (u.BN / 4) * 20);
        u.lds_bytes = (floats > (size_t)kWinoXchg ? floats : (size_t)kWinoXchg) * sizeof(float);
    }
    if (u.lds_bytes > 160 * 1024) return u;
    pc.magic_psz = div_magic((unsigned)pc.psz);
    pc.magic_img = div_magic((unsigned)(pc.PR * pc.PC));
    pc.magic_pc = div_magic((unsigned)pc.PC);
    pc.mtiles = (pc.Mout + BM - 1) / BM;
    pc.ntiles = (pc.ncols + BN - 1) / BN;
    pc.Mp = pc.mtiles * BM;
    pc.chunks_total = (pc.Cin + 15) / 16;
    pc.out_elems = (size_t)pc.ncols * pc.Mout;
    u.tiles = pc.mtiles * pc.ntiles;
    u.wp_elems = (size_t)pc.chunks_total * (wino ? 16 : 9) * pc.Mp * 16;
    u.ok = true;
    return u;
}

template <bool kBwd>
PackJob pack_job(const dopt_hip_conv_desc *d, const PatchSetup &u, const float *w, float *wp)
{
    const unsigned C9 = (unsigned)(d->C * 9);
    PackJob j{};
    j.w = w; j.wp = wp;
    j.M = u.pc.Mout; j.Cred = u.pc.Cin; j.Mp = u.pc.Mp; j.bwd = kBwd;
    j.wino = u.shape == 4; j.flip = u.pc.flip;
    j.sm = kBwd ? 9u : C9;
    j.sc = kBwd ? C9 : 9u;
    j.mblocks = (unsigned)(u.pc.Mp / 16);
    return j;
}

// How many ways to split the channel chunks of a patch convolution over blocks.  `slots` blocks run
// at once (one or two per CU); the blocks of a launch run in ceil(blocks / slots) rounds and a round
// lasts as long as one block, so 320 tiles on 256 slots cost two full rounds - unless the reduction
// is split four ways, which makes 1280 quarter-length blocks in exactly five rounds.  The estimate,
// in microseconds: rounds x (chunks per block x time per chunk + a fixed prologue/epilogue) plus,
// when split, writing and re-reading the partial tiles.  The split with the lowest estimate wins;
// ties go to the smaller one.
int patch_splits(int tiles, int chunks, int slots, int BM, int BN, size_t out_elems)
{
    const double cu_tflops = 0.47;                                   // what one CU sustains in these main loops
    const double per_cu = (double)slots / num_cus();                 // blocks sharing a CU
    const double t_chunk = 2.0 * BM * BN * 144 / (cu_tflops * 1e6 / per_cu);   // 16 channels x 9 taps
    int best = 1;
    double best_cost = 0.0;
    for (int sp = 1; sp <= chunks && sp <= 64; sp++) {
        const int per_block = (chunks + sp - 1) / sp;
        if (sp > 1 && (chunks + per_block - 1) / per_block != sp) continue;   // would leave an empty split
        const double rounds = (double)(((long long)tiles * sp + slots - 1) / slots);
        double cost = rounds * (per_block * t_chunk + 6.0);
        if (sp > 1) cost += 3.0 + (sp + 1.0) * out_elems * 4.0 / 4.5e6;       // partial tiles at ~4.5 TB/s
        if (sp == 1 || cost < best_cost * 0.97) {                    // a larger split must pay for itself clearly
            best = sp;
            best_cost = cost;
        }
    }
    return best;
}

// The same estimate for the general kernels, whose unit is a slab of 16 reduction steps and whose main loops
// sustain less (k-major LDS tiles, 32-bit fragment reads).
int gather_splits(int tiles, int slabs, int slots, int BM, int BN, size_t out_elems, int cap = 64)
{
    const double cu_tflops = 0.33;
    const double per_cu = (double)slots / num_cus();
    const double t_slab = 2.0 * BM * BN * 16 / (cu_tflops * 1e6 / per_cu);
    int best = 1;
    double best_cost = 0.0;
    for (int sp = 1; sp <= slabs && sp <= cap; sp++) {
        const int per_block = (slabs + sp - 1) / sp;
        if (sp > 1 && (slabs + per_block - 1) / per_block != sp) continue;
        const double rounds = (double)(((long long)tiles * sp + slots - 1) / slots);
        double cost = rounds * (per_block * t_slab + 6.0);
        if (sp > 1) cost += 3.0 + (sp + 1.0) * out_elems * 4.0 / 4.5e6;
        if (sp == 1 || cost < best_cost * 0.97) {
            best = sp;
            best_cost = cost;
        }
    }
    return best;
}

// Fills in how a patch convolution splits its channel chunks over blocks; returns the number of splits.
int patch_decide_splits(PatchSetup *u, const float *out)
{
    PatchConv &pc = u->pc;
    int splits = patch_splits(u->tiles, pc.chunks_total, u->blocks_wanted, u->BM, u->BN, pc.out_elems);
    if (pc.out_elems % 4 != 0 || !aligned16(out)) splits = 1;
    pc.chunks_per_split = (pc.chunks_total + splits - 1) / splits;
    splits = (pc.chunks_total + pc.chunks_per_split - 1) / pc.chunks_per_split;
    pc.splits = splits;
    return splits;
}

// `prepacked`: the filter already in the kernel's layout (dopt_hip_conv_pack_batch), or null to
// pack it here first.
// Device time of one kernel family alone (an entry point may also run split sums and packing): while the probe is on,
// every launch of the family - 1: the one-launch backward pairs (conv_bwd_pair_k), 2: the Winograd kernel
// (conv_wino_k) - is bracketed by two events on the stream it is launched on.
struct PairProbe {
    int on = 0;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> events;   // kept for the process's lifetime, reused
    size_t used = 0;
    double flops = 0.0, bytes = 0.0;
};
PairProbe g_pair_probe;

int probe_begin(PairProbe &probe)
{
    if (probe.used == probe.events.size()) {
        hipEvent_t e0, e1;
        DOPT_HIP_CHECK(hipEventCreate(&e0));
        DOPT_HIP_CHECK(hipEventCreate(&e1));
        probe.events.push_back({e0, e1});
    }
    DOPT_HIP_CHECK(hipEventRecord(probe.events[probe.used].first, stream()));
    return DOPT_HIP_OK;
}

// The launch of a filled-in patch setup: the tile shape picks the instance.
int dispatch_patch(const PatchSetup &u, int splits)
{
    const PatchConv &pc = u.pc;
    const dim3 grid(xcd_grid((unsigned)(u.tiles * splits)));
    const bool c_full = pc.Cin % 16 == 0;
    if (u.shape == 0) return launch_patch<GatherWide, 24>(pc, c_full, grid, u.lds_bytes);
    if (u.shape == 1) return launch_patch<GatherSquare, 16>(pc, c_full, grid, u.lds_bytes);
    if (u.shape == 3) return launch_patch<GatherTall, 16>(pc, c_full, grid, u.lds_bytes);
    if (u.shape == 4) {
        static bool raised = false;
        if (!raised) {
            DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)conv_wino_k<16, 4, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)conv_wino_k<16, 2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            raised = true;
        }
        PairProbe &probe = g_pair_probe;
        const bool probing = probe.on == 2 && u.BM == 128 && !capturing();   // the 128-row instantiation only: one kernel, one average
        if (probing)
            if (int rc = probe_begin(probe)) return rc;
        if (u.BM == 128) hipLaunchKernelGGL((conv_wino_k<16, 4, 1>), grid, dim3(512), u.lds_bytes, stream(), pc);
        else hipLaunchKernelGGL((conv_wino_k<16, 2, 2>), grid, dim3(512), u.lds_bytes, stream(), pc);
        DOPT_LAUNCH_CHECK();
        if (probing) {
            DOPT_HIP_CHECK(hipEventRecord(probe.events[probe.used++].second, stream()));
            // the direct algorithm's count (what the layer is, whatever the kernel multiplies): 2 N K C 9 P Q
            probe.flops += 2.0 * (double)pc.ncols * pc.Mout * pc.Cin * 9.0;
            probe.bytes += 4.0 * ((double)pc.N * pc.Cin * pc.IH * pc.IW + (double)pc.ncols * pc.Mout + (double)pc.Mout * pc.Cin * 9.0);
        }
        return DOPT_HIP_OK;
    }
    return launch_patch<GatherDeep, 16>(pc, c_full, grid, u.lds_bytes);
}

template <bool kBwd>
int run_patch(const dopt_hip_conv_desc *d, size_t P, size_t Q, const float *in, const float *w, const float *bias,
              float *out, bool *done, const float *prepacked = nullptr, dopt_hip_split_sum *open = nullptr)
{
    *done = false;
    PatchSetup u = patch_setup<kBwd>(d, P, Q);
    if (!u.ok) return DOPT_HIP_OK;
    PatchConv &pc = u.pc;
    const int tiles = u.tiles;
    const int splits = patch_decide_splits(&u, out);

    const size_t wp_bytes = prepacked ? 0 : (u.wp_elems * sizeof(float) + 255) / 256 * 256;
    const size_t part_bytes = splits > 1 ? (size_t)splits * pc.out_elems * sizeof(float) : 0;
    char *ws = wp_bytes + part_bytes > 0 ? (char *)workspace(wp_bytes + part_bytes) : nullptr;
    if (wp_bytes + part_bytes > 0 && !ws) return DOPT_HIP_ERR_OOM;
    float *partial = (float *)(ws + wp_bytes);
    if (!prepacked) {
        const PackJob j = pack_job<kBwd>(d, u, w, (float *)ws);
        const dim3 pgrid(j.mblocks, (unsigned)pc.chunks_total);
        if (!kBwd) hipLaunchKernelGGL(pack_patch_k<false>, pgrid, dim3(256), 0, stream(), j.M, j.Cred, j.Mp, (size_t)j.sm,
                                      (size_t)j.sc, j.wino, j.flip, w, j.wp);
        else hipLaunchKernelGGL(pack_patch_k<true>, pgrid, dim3(256), 0, stream(), j.M, j.Cred, j.Mp, (size_t)j.sm,
                                (size_t)j.sc, j.wino, j.flip, w, j.wp);
        DOPT_LAUNCH_CHECK();
        prepacked = j.wp;
    }
    pc.in = in;
    pc.wp = prepacked;
    pc.bias = bias;
    pc.in_bytes = (size_t)pc.N * pc.Cin * pc.IH * pc.IW * sizeof(float);
    pc.wp_bytes = u.wp_elems * sizeof(float);
    pc.out = splits > 1 ? partial : out;
    if (int rc = dispatch_patch(u, splits)) return rc;
    *done = true;
    if (splits > 1 && open) {   // the caller's next call adds the copies
        open->partial = partial;
        open->splits = splits;
        open->elems = pc.out_elems;
        open->C = (size_t)pc.Mout;
        open->inner = (size_t)pc.OH * pc.OW;
        open->bias = bias;
        open->value = out;
        open_split_set(partial);
        return DOPT_HIP_OK;
    }
    if (splits > 1)
        return launch_splitk_reduce(pc.out_elems, splits, partial, out, bias, (unsigned)pc.Mout, (unsigned)(pc.OH * pc.OW));
    return DOPT_HIP_OK;
}

// ---- 2 x 2 images -------------------------------------------------------------------------------
// On a 2 x 2 image with pad 1 every output pixel sees every input pixel, each through exactly one
// tap, and the five taps that fall on padding contribute nothing.  The convolution is then a plain
// product of the batch, flattened [N, C*4], with a [C*4, K*4] matrix built from the filter:
//     Wd[(c, iy, ix)][(k, oy, ox)] = w[k][c][2 - (iy - oy + 1)][2 - (ix - ox + 1)]
// (the flipped filter, core/source/dopt/core/ops/nnet.d:270-293) - 4/9 of the multiplications of
// the nine-tap form.  NCHW needs no rearranging on either side, forward is x * Wd and backward-data
// is dy * Wd^T, so one copy of Wd serves both directions.
__global__ __launch_bounds__(256) void pack_2x2_k(unsigned C, unsigned K, const float *w, float4 *wd)
{
    // A block takes 8 output channels x 64 input channels.  It reads their filter planes as eight
    // contiguous runs of 64 x 9 floats, and after a pass through LDS writes, for each of the 256
    // (input channel, input pixel) rows, the eight quads of its output channels: one full 128-byte line.
    __shared__ float stage[8][64 * 9 + 1];
    const unsigned k0 = blockIdx.x * 8, c0 = blockIdx.y * 64;
    const unsigned nk = min(8u, K - k0), nc = min(64u, C - c0);
    float v[18];   // 8 * 64 * 9 / 256 loads per thread, all issued before the first is used (clamped, not branched)
#pragma unroll
    for (int u = 0; u < 18; u++) {
        const unsigned i = threadIdx.x + 256 * u, kk = i / (64 * 9), r = i - kk * (64 * 9);
        v[u] = w[((size_t)(k0 + min(kk, nk - 1)) * C + c0) * 9 + min(r, nc * 9 - 1)];
    }
#pragma unroll
    for (int u = 0; u < 18; u++) {
        const unsigned i = threadIdx.x + 256 * u, kk = i / (64 * 9), r = i - kk * (64 * 9);
        stage[kk][r] = v[u];   // rows and channels past the end are never read back
    }
    __syncthreads();
    for (unsigned i = threadIdx.x; i < 64 * 4 * 8; i += 256) {
        const unsigned kk = i & 7, row = i >> 3, cc = row >> 2, iy = (row >> 1) & 1, ix = row & 1;
        if (kk >= nk || cc >= nc) continue;
        // input pixel (iy, ix), output pixel (oy, ox): tap (1 - iy + oy, 1 - ix + ox)
        const float *f = &stage[kk][cc * 9 + (1 - iy) * 3 + (1 - ix)];
        wd[((size_t)(c0 + cc) * 4 + iy * 2 + ix) * K + k0 + kk] = make_float4(f[0], f[1], f[3], f[4]);
    }
}

bool dense2x2_takes(const dopt_hip_conv_desc *d)
{
    return d->R == 3 && d->S == 3 && d->strideH == 1 && d->strideW == 1 && d->padH == 1 && d->padW == 1 && d->H == 2 &&
           d->W == 2 && d->C * 4 < ((size_t)1 << 30) && d->K * 4 < ((size_t)1 << 30);
}

size_t dense2x2_elems(const dopt_hip_conv_desc *d) { return (size_t)16 * d->C * d->K; }

int dense2x2_pack(const dopt_hip_conv_desc *d, const float *w, float *wd)
{
    hipLaunchKernelGGL(pack_2x2_k, dim3((unsigned)ceil_div(d->K, (size_t)8), (unsigned)ceil_div(d->C, (size_t)64)), dim3(256), 0,
                       stream(), (unsigned)d->C, (unsigned)d->K, w, (float4 *)wd);   // pool and plan buffers are 256-byte aligned
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// `wd`: the matrix already built, or null to build it from `w` in the workspace first
template <bool kBwd>
int run_dense2x2(const dopt_hip_conv_desc *d, const float *in, const float *w, const float *wd, const float *bias,
                 float *out)
{
    void *mine = nullptr;   // from the pool, not the workspace: the product below may use the workspace itself
    if (!wd) {
        if (int rc = scratch_alloc(&mine, dense2x2_elems(d) * sizeof(float))) return rc;
        if (int rc = dense2x2_pack(d, w, (float *)mine)) {
            dopt_hip_free(mine);
            return rc;
        }
        wd = (const float *)mine;
    }
    bool biased = false;
    int rc;
    if (!kBwd) {
        rc = sgemm_bias(0, 0, d->N, 4 * d->K, 4 * d->C, in, wd, out, bias, 2, &biased);
        if (!rc && bias && !biased) rc = dopt_hip_bias_fwd(d->N, d->K, 4, out, bias, out);
    } else {
        rc = sgemm_bias(0, 1, d->N, 4 * d->C, 4 * d->K, in, wd, out, nullptr, 0, &biased);
    }
    if (mine) dopt_hip_free(mine);   // back to the pool; whoever gets it next queues behind the product
    return rc;
}

// ---- 2 x 2 images, straight from the filter ----------------------------------------------------
// The product above needs the 16 MB matrix made first, and its 32 x 32-output blocks read their operands
// with a handful of loads in flight per wavefront (one cache line per lane and step), which is what
// bounds them.  This kernel keeps that decomposition - a block owns 32 images x 8 output channels x 4
// pixels over the WHOLE reduction, so nothing is split and no partial copies are left for a reader
// (whose 16-byte pieces per image and channel would be re-read once per copy) - but reads the taps from
// the filter as it lies (no Wd) and streams both operands through LDS in bulk:
//   * the eight wavefronts split the reduction channels (64 consecutive channels each, R % 64 == 0) and
//     never share data, so each runs a pipeline of its own with no workgroup barrier: per step of 8
//     channels it loads 32 images x 128 bytes of the batch (whole cache lines) and 8 runs of 8 x 9 taps,
//     three steps ahead, passes them through a wavefront-private LDS tile and multiplies;
//   * a batch row is read back as one 128-bit LDS read per eight reduction steps (lane half h takes
//     steps 8g + 4h .. 8g + 4h + 3 on both operands), the four taps a lane needs per (channel, pixel
//     pair) as four 4-byte reads: tap = {4,3,1,0}[input pixel] + {0,1,3,4}[output pixel] (see Wd above);
//   * the eight partial 32 x 32 tiles are added through LDS in wavefront order (+ bias).
// Forward (kBwd = false): in = x [N][C*4], columns (k, output pixel), a filter run = one output channel's
// 8 reduction channels x 9 taps; backward-data: in = dy [N][K*4], columns (c, input pixel), a run = one
// reduction channel k, its 8 output channels c x 9 taps.
struct Direct2x2 {
    const float *in;    // [N][R*4]
    const float *w;     // [K][C][3][3]
    const float *bias;  // [O] or null (forward)
    float *out;         // [N][O*4]
    int N, R, O, C;     // images, reduction channels, output channels, the filter's input channels (its pitch is C*9)
};

constexpr int kD2Rows = 32, kD2Chans = 8, kD2Step = 8, kD2Waves = 8, kD2Depth = 3;
constexpr int kD2APitch = kD2Step * 4 + 4;   // 36 floats: 128-bit reads of 32 rows touch every bank once
constexpr int kD2WPitch = kD2Step * 9 + 5;   // 77 floats per run of 8 x 9 taps
constexpr int kD2WaveLds = 2 * (kD2Rows * kD2APitch + 8 * kD2WPitch);   // floats per wavefront, double buffered
constexpr size_t kD2Lds = (size_t)kD2Waves * kD2WaveLds * sizeof(float);
static_assert(kD2Waves * kD2WaveLds >= kD2Waves * 32 * 33, "the partial tiles reuse the staging area");

template <bool kBwd>
__global__ __launch_bounds__(64 * kD2Waves) void conv2x2_direct_k(Direct2x2 p)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, l32 = lane & 31, kh = lane >> 5;
    const int o0 = blockIdx.x * kD2Chans, n0 = blockIdx.y * kD2Rows;
    const int per_wave = p.R / kD2Waves, steps = per_wave / kD2Step, c_first = w * per_wave;
    float *const mine = lds + w * kD2WaveLds;

    // this lane's pieces of a step: 4 quads of the batch (row = idx / 8, quad idx % 8) and up to 3 of the taps
    // (run = idx / 18, quad idx % 18)
    const float *a_src[4];
    bool a_ok[4];
    int a_dst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int idx = lane + 64 * i, row = idx >> 3, q = idx & 7;
        a_ok[i] = n0 + row < p.N;
        a_src[i] = p.in + ((size_t)(a_ok[i] ? n0 + row : 0) * p.R + c_first) * 4 + 4 * q;
        a_dst[i] = row * kD2APitch + 4 * q;
    }
    const float *w_src[3];
    bool w_ok[3];
    int w_dst[3];
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const int idx = lane + 64 * i, run = min(idx / 18, 7), q = idx - (idx / 18) * 18;
        w_ok[i] = idx < 8 * 18;
        // forward: run = output channel, its 8 reduction channels of the step; backward: run = reduction channel of the
        // step, the block's 8 output channels
        w_src[i] = kBwd ? p.w + ((size_t)(c_first + run) * p.C + o0) * 9 + 4 * q : p.w + ((size_t)(o0 + run) * p.C + c_first) * 9 + 4 * q;
        w_dst[i] = run * kD2WPitch + 4 * q;
    }
    const size_t w_step = kBwd ? (size_t)kD2Step * p.C * 9 : (size_t)kD2Step * 9;   // floats between steps
    float4 ra[kD2Depth][4], rw[kD2Depth][3];
    auto load = [&](int slot, int s) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            ra[slot][i] = a_ok[i] ? *(const float4 *)(a_src[i] + (size_t)s * kD2Step * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 3; i++)
            rw[slot][i] = w_ok[i] ? *(const float4 *)(w_src[i] + (size_t)s * w_step) : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    auto store = [&](int slot, float *buf) {
        float *As = buf, *Ws = buf + kD2Rows * kD2APitch;
#pragma unroll
        for (int i = 0; i < 4; i++) *(float4 *)&As[a_dst[i]] = ra[slot][i];
#pragma unroll
        for (int i = 0; i < 3; i++)
            if (w_ok[i]) {
                float *dst = &Ws[w_dst[i]];
                dst[0] = rw[slot][i].x; dst[1] = rw[slot][i].y; dst[2] = rw[slot][i].z; dst[3] = rw[slot][i].w;
            }
    };

    const int pix = l32 & 3, oc = l32 >> 2;   // the column: output channel inside the block, and its pixel
    const int lane_tap = kBwd ? (pix == 0 ? 4 : pix == 1 ? 3 : pix == 2 ? 1 : 0) : (pix == 0 ? 0 : pix == 1 ? 1 : pix == 2 ? 3 : 4);
    const int a_frag = l32 * kD2APitch + 4 * kh;
    const int b_frag = kD2Rows * kD2APitch + (kBwd ? kh * kD2WPitch + oc * 9 + lane_tap : oc * kD2WPitch + kh * 9 + lane_tap);
    // two accumulators (even and odd channel pairs), so that consecutive matrix instructions do not wait for each other
    v16f acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; v++) acc0[v] = acc1[v] = 0.0f;

#pragma unroll
    for (int d = 0; d < kD2Depth; d++)
        if (d < steps) load(d, d);
    // steps in groups of kD2Depth so that the register slots are compile-time indices
    for (int s0 = 0; s0 < steps; s0 += kD2Depth) {
#pragma unroll
        for (int d = 0; d < kD2Depth; d++) {
            const int s = s0 + d;
            if (s < steps) {
                float *buf = mine + (s & 1) * (kD2WaveLds / 2);
                store(d, buf);
                __builtin_amdgcn_wave_barrier();   // the tile is read by other lanes of this wavefront: keep the order
                if (s + kD2Depth < steps) load(d, s + kD2Depth);
#pragma unroll
                for (int g = 0; g < 4; g++) {   // reduction steps 8g .. 8g + 7 of the tile: channels 2g (lane half 0), 2g + 1
                    const float4 a = *(const float4 *)(buf + a_frag + 8 * g);
                    const float *src = buf + b_frag + (kBwd ? 2 * g * kD2WPitch : 2 * g * 9);
                    float b0, b1, b2, b3;
                    if (kBwd) { b0 = src[0]; b1 = src[1]; b2 = src[3]; b3 = src[4]; }
                    else { b0 = src[4]; b1 = src[3]; b2 = src[1]; b3 = src[0]; }
                    if (g & 1) {
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b0, acc1, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b1, acc1, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b2, acc1, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b3, acc1, 0, 0, 0);
                    } else {
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b0, acc0, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b1, acc0, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b2, acc0, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b3, acc0, 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- the eight partial tiles, added in wavefront order
    __syncthreads();   // every wavefront is done with its staging tiles
    float *red = lds;  // [8][32 * 33]
#pragma unroll
    for (int v = 0; v < 16; v++) red[w * (32 * 33) + acc_row(v, lane) * 33 + l32] = acc0[v] + acc1[v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int idx = tid + i * 64 * kD2Waves, rr = idx >> 5, cc = idx & 31;
        float sum = red[rr * 33 + cc];
#pragma unroll
        for (int k = 1; k < kD2Waves; k++) sum += red[k * (32 * 33) + rr * 33 + cc];
        if (p.bias) sum += p.bias[o0 + (cc >> 2)];
        if (n0 + rr < p.N) p.out[(size_t)(n0 + rr) * p.O * 4 + o0 * 4 + cc] = sum;
    }
}

bool direct2x2_takes(const dopt_hip_conv_desc *d)
{
    return dense2x2_takes(d) && d->C % 64 == 0 && d->K % 64 == 0 && d->N * d->C * 4 < ((size_t)1 << 31) &&
           d->N * d->K * 4 < ((size_t)1 << 31) && d->K * d->C * 9 < ((size_t)1 << 31) && ceil_div(d->N, (size_t)kD2Rows) < 65536;
}

// *done = false: not this kernel's shape (or operands it cannot read as quads).
template <bool kBwd>
int run_direct2x2(const dopt_hip_conv_desc *d, const float *in, const float *w, const float *bias, float *out, bool *done)
{
    *done = false;
    if (!direct2x2_takes(d) || !aligned16(in) || !aligned16(w) || !aligned16(out)) return DOPT_HIP_OK;
    Direct2x2 p{};
    p.in = in;
    p.w = w;
    p.bias = bias;
    p.out = out;
    p.N = (int)d->N;
    p.R = (int)(kBwd ? d->K : d->C);
    p.O = (int)(kBwd ? d->C : d->K);
    p.C = (int)d->C;
    static bool raised[2] = {false, false};
    if (!raised[kBwd]) {
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)conv2x2_direct_k<kBwd>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kD2Lds));
        raised[kBwd] = true;
    }
    // column tiles fastest: the blocks an XCD receives share an eighth of the filter and all of the batch
    const dim3 grid((unsigned)(p.O / kD2Chans), (unsigned)ceil_div(d->N, (size_t)kD2Rows));
    hipLaunchKernelGGL(conv2x2_direct_k<kBwd>, grid, dim3(64 * kD2Waves), kD2Lds, stream(), p);
    DOPT_LAUNCH_CHECK();
    *done = true;
    return DOPT_HIP_OK;
}

// Filter gradient of the same layers: dWd = x^T * dy, [4C, N] x [N, 4K], is the gradient of the matrix
// above; every filter tap collects the (input pixel, output pixel) pairs that read it - one pair for
// a corner tap, two for an edge tap, four for the centre - in a fixed order.
__global__ __launch_bounds__(256) void fold_2x2_k(unsigned C, unsigned K, const float4 *dwd, float *dw)
{
    const size_t total = (size_t)C * K;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const unsigned k = (unsigned)(i % K), c = (unsigned)(i / K);
        float q[4][4];   // [input pixel iy*2+ix][output pixel oy*2+ox]
#pragma unroll
        for (int pin = 0; pin < 4; pin++) {
            const float4 v = dwd[((size_t)c * 4 + pin) * K + k];
            q[pin][0] = v.x; q[pin][1] = v.y; q[pin][2] = v.z; q[pin][3] = v.w;
        }
        float *out = dw + ((size_t)k * C + c) * 9;
#pragma unroll
        for (int a = 0; a < 3; a++)
#pragma unroll
            for (int b = 0; b < 3; b++) {
                float sum = 0.0f;   // pairs with 1 - iy + oy == a and 1 - ix + ox == b
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

int run_dense2x2_wgrad(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw)
{
    int rc = DOPT_HIP_OK;
    if (sgemm_fold2x2(d->C, d->K, d->N, x, dy, dw, &rc)) return rc;   // product and fold in one kernel
    void *dwd = nullptr;
    if ((rc = scratch_alloc(&dwd, dense2x2_elems(d) * sizeof(float)))) return rc;
    bool biased = false;
    rc = sgemm_bias(1, 0, 4 * d->C, 4 * d->K, d->N, x, dy, (float *)dwd, nullptr, 0, &biased);
    if (!rc) {
        const size_t blocks = ceil_div(d->C * d->K, (size_t)256);
        const size_t cap = (size_t)num_cus() * 16;
        hipLaunchKernelGGL(fold_2x2_k, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0, stream(), (unsigned)d->C,
                           (unsigned)d->K, (const float4 *)dwd, dw);
        if (hipGetLastError() != hipSuccess) rc = fail(DOPT_HIP_ERR_RUNTIME, "convolution: fold launch failed");
    }
    dopt_hip_free(dwd);
    return rc;
}

// Packs the filter w[K][C][g.R * g.S] and runs conv_gather_k on a problem whose geometry the caller
// has filled in (dimensions, padding, stride, output placement).  mode as conv_gather_k's kMode.
int gather_launch(GatherConv g, int mode, int K, int C, const float *in, const float *w, float *out)
{
    const bool bwd = mode != 0;
    const int taps = g.R * g.S;
    g.CinPad = round_up(g.Cin, BK);
    g.Mp = round_up(g.Mout, 4);
    g.ncols = g.N * g.OH * g.OW;
    g.slabs_total = taps * g.CinPad / BK;
    g.out_elems = (size_t)g.ncols * g.Mout;
    const bool dense = g.out_sy == 1 && g.out_sx == 1 && g.out_plane == g.OH * g.OW;

    // tile shape: 64-row tiles for <= 64 output channels and wherever 128-row tiles would pad more;
    // otherwise 128x128, with 8 wavefronts per workgroup when there are too few tiles to give every
    // CU two 4-wavefront workgroups
    enum { kWide, kSquare, kDeep } shape;
    int BM, BN, blocks_wanted;
    if (g.Mout <= 64 || (g.Mout + 63) / 64 * 64 < (g.Mout + 127) / 128 * 128) {
        shape = kWide; BM = 64; BN = 256; blocks_wanted = 2 * num_cus();
    } else {
        BM = 128; BN = 128;
        const int t = ((g.Mout + 127) / 128) * ((g.ncols + 127) / 128);
        if (t >= 2 * num_cus()) { shape = kSquare; blocks_wanted = 2 * num_cus(); }
        else { shape = kDeep; blocks_wanted = num_cus(); }
    }
    g.mtiles = (g.Mout + BM - 1) / BM;
    g.ntiles = (g.ncols + BN - 1) / BN;
    const int tiles = g.mtiles * g.ntiles;
    int splits = gather_splits(tiles, g.slabs_total, blocks_wanted, BM, BN, g.out_elems);
    // the split reduction works on float4 over a dense output
    if (g.out_elems % 4 != 0 || !aligned16(out) || !dense) splits = 1;
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
    if (g.CinPad != g.Cin || g.Mp != g.Mout) {
        if (capturing()) return fail(DOPT_HIP_ERR_UNSUPPORTED, "convolution: a fill cannot be recorded into a graph");
        DOPT_HIP_CHECK(hipMemsetAsync(wp, 0, wp_elems * sizeof(float), stream()));
    }
    if (!bwd) {
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
#define DOPT_GATHER(TILE)                                                                                      \
    do {                                                                                                       \
        if (mode == 0) hipLaunchKernelGGL((conv_gather_k<TILE, 0>), grid, dim3(TILE::THREADS), 0, stream(), g); \
        else if (mode == 1) hipLaunchKernelGGL((conv_gather_k<TILE, 1>), grid, dim3(TILE::THREADS), 0, stream(), g); \
        else hipLaunchKernelGGL((conv_gather_k<TILE, 2>), grid, dim3(TILE::THREADS), 0, stream(), g);          \
    } while (0)
    if (shape == kWide) DOPT_GATHER(GatherWide);
    else if (shape == kSquare) DOPT_GATHER(GatherSquare);
    else DOPT_GATHER(GatherDeep);
#undef DOPT_GATHER
    DOPT_LAUNCH_CHECK();
    if (splits > 1) return launch_splitk_reduce(g.out_elems, splits, partial, out);
    return DOPT_HIP_OK;
}

// ---- backward-data with a stride, one residue class of output pixels at a time -------------------
// dx[n, c, h, w] = sum over k, r, s with (h + padH - r) and (w + padW - s) multiples of the stride of
// dy[n, k, (h + padH - r) / sH, (w + padW - s) / sW] * w[k, c, R - 1 - r, S - 1 - s] (the flipped filter).  Which taps qualify depends only
// on (h mod sH, w mod sW).  Taking all pixels together (conv_gather_k mode 2) multiplies every pixel
// by every tap and masks three quarters of the products of a stride-2 3x3 layer; taking the pixels
// of one class (a, b) = (h mod sH, w mod sW) at a time, only its taps r = r0, r0 + sH, ... and s = s0,
// s0 + sW, ... are multiplied, and the class is a UNIT-stride problem on the grid (i, j) = (h / sH, w / sW):
//     dy row = i + (a + padH - r0) / sH - t   for its t-th tap row,
// i.e. backward-data of a filter with ceil((R - r0) / sH) rows, padding (a + padH - r0) / sH and rows
// stored in reverse order of r.  The sub-filter is copied out of w, the kernel's output placement
// scatters the class back into dx.
__global__ __launch_bounds__(256) void subfilter_k(int KC, int R, int S, int R2, int S2, int r0, int s0, int sH, int sW,
                                                    const float *w, float *sub)
{
    const int total = KC * R2 * S2;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
        const int kc = i / (R2 * S2), t = i - kc * (R2 * S2), tr = t / S2, ts = t - tr * S2;
        // stored row tr of the sub-filter stands for tap offset r = r0 + (R2 - 1 - tr) * sH, and the filter
        // element that multiplies offset r is the flipped one, w[.., R - 1 - r, S - 1 - s]
        const int r = r0 + (R2 - 1 - tr) * sH, sc = s0 + (S2 - 1 - ts) * sW;
        sub[i] = w[(size_t)kc * (R * S) + (R - 1 - r) * S + (S - 1 - sc)];
    }
}

// The packed sub-filters of all classes in one launch: block (k, 64-channel chunk) stages w[k][c0 .. c0+64][*]
// once and writes each class's taps as pack_bwd_k would write them from that class's sub-filter.
struct SubFilter {
    float *wp;            // [(tap * KPad + k)][Mp] of this class
    int R2, S2, r0, s0;   // tap rows / columns of the class and its first tap offsets
};
struct SubFilters {
    SubFilter f[kGatherJobs];
    int n;
};
__global__ __launch_bounds__(256) void pack_bwd_classes_k(int K, int C, int R, int S, int sH, int sW, int KPad, int Mp,
                                                           const float *w, SubFilters subs)
{
    extern __shared__ float stage[];  // 64 * R * S floats
    const int k = blockIdx.x, c0 = blockIdx.y * 64, RS = R * S;
    const int nc = min(64, C - c0);
    const float *src = w + ((size_t)k * C + c0) * RS;
    for (int i = threadIdx.x; i < nc * RS; i += 256) stage[i] = src[i];
    __syncthreads();
    for (int j = 0; j < subs.n; j++) {
        const SubFilter f = subs.f[j];
        const int taps = f.R2 * f.S2;
        for (int i = threadIdx.x; i < nc * taps; i += 256) {
            const int t = i / nc, c = i - t * nc, tr = t / f.S2, ts = t - tr * f.S2;
            // stored tap (tr, ts) stands for offsets r = r0 + (R2 - 1 - tr) * sH, s likewise, and the element
            // that multiplies offset (r, s) is the flipped one (see subfilter_k)
            const int r = f.r0 + (f.R2 - 1 - tr) * sH, sc = f.s0 + (f.S2 - 1 - ts) * sW;
            f.wp[(size_t)(t * KPad + k) * Mp + c0 + c] = stage[c * RS + (R - 1 - r) * S + (S - 1 - sc)];
        }
    }
}

int run_bwd_strided(const dopt_hip_conv_desc *d, size_t P, size_t Q, const float *dy, const float *w, float *dx)
{
    const int sH = (int)d->strideH, sW = (int)d->strideW, R = (int)d->R, S = (int)d->S;
    const int H = (int)d->H, W = (int)d->W, padH = (int)d->padH, padW = (int)d->padW;
    struct Cls { int n, first, taps, pad; };   // pixels of the class along one axis, its first tap, tap count, padding
    auto cls = [](int a, int extent, int stride, int pad, int filt) {
        Cls c{};
        c.n = a < extent ? (extent - a + stride - 1) / stride : 0;
        c.first = (a + pad) % stride;
        c.taps = c.first < filt ? (filt - c.first + stride - 1) / stride : 0;
        c.pad = (a + pad - c.first) / stride;
        return c;
    };
    bool gaps = false;   // classes no tap reaches: those pixels of dx are zero
    for (int a = 0; a < sH; a++) gaps = gaps || (cls(a, H, sH, padH, R).n > 0 && cls(a, H, sH, padH, R).taps == 0);
    for (int b = 0; b < sW; b++) gaps = gaps || (cls(b, W, sW, padW, S).n > 0 && cls(b, W, sW, padW, S).taps == 0);
    if (gaps)
        if (int rc = dopt_hip_memset(dx, 0, d->N * d->C * d->H * d->W * sizeof(float))) return rc;
    // Two to nine classes with work (a 3 x 3 filter at stride 2 has four: 1, 2, 2 and 4 taps): one launch packs all
    // their sub-filters and one launch multiplies all of them, instead of three dependent launches per class.
    struct Job { Cls ch, cw; int a, b; };
    Job jobs[kGatherJobs];
    int njobs = 0;
    bool fits = true;
    for (int a = 0; a < sH; a++)
        for (int b = 0; b < sW; b++) {
            const Cls ch = cls(a, H, sH, padH, R), cw = cls(b, W, sW, padW, S);
            if (ch.n == 0 || cw.n == 0 || ch.taps == 0 || cw.taps == 0) continue;
            if (njobs == kGatherJobs) { fits = false; continue; }
            jobs[njobs++] = Job{ch, cw, a, b};
        }
    if (fits && njobs >= 2) {
        for (int i = 1; i < njobs; i++)   // most taps first (insertion sort, stable)
            for (int j = i; j > 0 && jobs[j].ch.taps * jobs[j].cw.taps > jobs[j - 1].ch.taps * jobs[j - 1].cw.taps; j--)
                std::swap(jobs[j], jobs[j - 1]);
        const int K = (int)d->K, C = (int)d->C;
        const int KPad = round_up(K, BK), Mp = round_up(C, 4);
        size_t wp_off[kGatherJobs + 1] = {0};
        for (int j = 0; j < njobs; j++) {
            const size_t elems = (size_t)jobs[j].ch.taps * jobs[j].cw.taps * KPad * Mp;
            wp_off[j + 1] = wp_off[j] + (elems * sizeof(float) + 255) / 256 * 256;
        }
        char *ws = (char *)workspace(wp_off[njobs]);
        if (!ws) return DOPT_HIP_ERR_OOM;
        if (KPad != K || Mp != C) {
            if (capturing()) return fail(DOPT_HIP_ERR_UNSUPPORTED, "convolution: a fill cannot be recorded into a graph");
            DOPT_HIP_CHECK(hipMemsetAsync(ws, 0, wp_off[njobs], stream()));
        }
        const bool wide = C <= 64 || (C + 63) / 64 * 64 < (C + 127) / 128 * 128;
        const int BM = wide ? 64 : 128, BN = wide ? 256 : 128;
        SubFilters subs{};
        GatherGroup gg{};
        subs.n = gg.n = njobs;
        unsigned blocks = 0, tiles_all = 0;
        for (int j = 0; j < njobs; j++) {
            const Job &jb = jobs[j];
            subs.f[j] = SubFilter{(float *)(ws + wp_off[j]), jb.ch.taps, jb.cw.taps, jb.ch.first, jb.cw.first};
            GatherConv &g = gg.g[j];
            g.N = (int)d->N;
            g.R = jb.ch.taps; g.S = jb.cw.taps;
            g.padH = jb.ch.pad; g.padW = jb.cw.pad;
            g.strideH = g.strideW = 1;
            g.Cin = K; g.IH = (int)P; g.IW = (int)Q;
            g.Mout = C; g.OH = jb.ch.n; g.OW = jb.cw.n;
            g.out_plane = H * W; g.out_OW = W;
            g.out_sy = sH; g.out_sx = sW; g.out_oy = jb.a; g.out_ox = jb.b;
            g.CinPad = KPad;
            g.Mp = Mp;
            g.ncols = g.N * g.OH * g.OW;
            g.slabs_total = g.R * g.S * KPad / BK;
            g.slabs_per_split = g.slabs_total;
            g.splits = 1;   // a class's pixels are scattered over dx: nothing for a split sum to add in place
            g.out_elems = (size_t)g.ncols * g.Mout;
            g.mtiles = (g.Mout + BM - 1) / BM;
            g.ntiles = (g.ncols + BN - 1) / BN;
            g.in = dy;
            g.wp = subs.f[j].wp;
            g.out = dx;
            g.in_bytes = (size_t)g.N * g.Cin * g.IH * g.IW * sizeof(float);
            g.wp_bytes = (size_t)g.R * g.S * KPad * Mp * sizeof(float);
            gg.per[j] = ((unsigned)(g.mtiles * g.ntiles) + 7u) / 8u;
            blocks += 8u * gg.per[j];
            tiles_all += (unsigned)(g.mtiles * g.ntiles);
        }
        hipLaunchKernelGGL(pack_bwd_classes_k, dim3((unsigned)K, (unsigned)((C + 63) / 64)), dim3(256),
                           (size_t)64 * R * S * sizeof(float), stream(), K, C, R, S, sH, sW, KPad, Mp, w, subs);
        DOPT_LAUNCH_CHECK();
        if (wide)
            hipLaunchKernelGGL((conv_gather_group_k<GatherWide, 1>), dim3(blocks), dim3(GatherWide::THREADS), 0, stream(), gg);
        else if (tiles_all >= 2u * (unsigned)num_cus())
            hipLaunchKernelGGL((conv_gather_group_k<GatherSquare, 1>), dim3(blocks), dim3(GatherSquare::THREADS), 0, stream(), gg);
        else
            hipLaunchKernelGGL((conv_gather_group_k<GatherDeep, 1>), dim3(blocks), dim3(GatherDeep::THREADS), 0, stream(), gg);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    void *sub = nullptr;
    if (int rc = scratch_alloc(&sub, d->K * d->C * d->R * d->S * sizeof(float))) return rc;
    int rc = DOPT_HIP_OK;
    for (int a = 0; a < sH && !rc; a++)
        for (int b = 0; b < sW && !rc; b++) {
            const Cls ch = cls(a, H, sH, padH, R), cw = cls(b, W, sW, padW, S);
            if (ch.n == 0 || cw.n == 0 || ch.taps == 0 || cw.taps == 0) continue;
            const int KC = (int)(d->K * d->C);
            hipLaunchKernelGGL(subfilter_k, dim3((unsigned)ceil_div((size_t)KC * ch.taps * cw.taps, (size_t)256)), dim3(256), 0,
                               stream(), KC, R, S, ch.taps, cw.taps, ch.first, cw.first, sH, sW, w, (float *)sub);
            if (hipGetLastError() != hipSuccess) {
                rc = fail(DOPT_HIP_ERR_RUNTIME, "convolution: sub-filter launch failed");
                break;
            }
            GatherConv g{};
            g.N = (int)d->N;
            g.R = ch.taps; g.S = cw.taps;
            g.padH = ch.pad; g.padW = cw.pad;
            g.strideH = g.strideW = 1;
            g.Cin = (int)d->K; g.IH = (int)P; g.IW = (int)Q;
            g.Mout = (int)d->C; g.OH = ch.n; g.OW = cw.n;
            g.out_plane = H * W; g.out_OW = W;
            g.out_sy = sH; g.out_sx = sW; g.out_oy = a; g.out_ox = b;
            rc = gather_launch(g, 1, (int)d->K, (int)d->C, dy, (const float *)sub, dx);
        }
    dopt_hip_free(sub);
    return rc;
}

// Shared host driver of forward (kBwd = false) and backward-data (kBwd = true).
template <bool kBwd>
int run_gather(const dopt_hip_conv_desc *d, size_t P, size_t Q, const float *in, const float *w, float *out,
               const float *bias = nullptr)
{
    if (!kBwd) {
        bool done = false;
        if (int rc = conv_smallc_fwd(d, in, w, bias, out, &done)) return rc;
        if (done) return DOPT_HIP_OK;
    }
    if (dense2x2_takes(d)) {
        bool done = false;
        if (int rc = run_direct2x2<kBwd>(d, in, w, bias, out, &done)) return rc;
        if (done) return DOPT_HIP_OK;
        return run_dense2x2<kBwd>(d, in, w, nullptr, bias, out);
    }
    {
        bool done = false;
        if (int rc = run_patch<kBwd>(d, P, Q, in, w, bias, out, &done)) return rc;
        if (done) return DOPT_HIP_OK;
    }
    if (bias) {  // the generic kernel has no fused bias: add it in place afterwards
        if (int rc = run_gather<kBwd>(d, P, Q, in, w, out, nullptr)) return rc;
        return dopt_hip_bias_fwd(d->N, kBwd ? d->C : d->K, kBwd ? d->H * d->W : P * Q, out, bias, out);
    }
    if (kBwd && (d->strideH > 1 || d->strideW > 1)) return run_bwd_strided(d, P, Q, in, w, out);
    GatherConv g{};
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
    g.out_plane = g.OH * g.OW;
    g.out_OW = g.OW;
    g.out_sy = g.out_sx = 1;
    return gather_launch(g, kBwd ? 1 : 0, (int)d->K, (int)d->C, in, w, out);
}

template <int WM, int WC, int kGeo>
int launch_wgrad_patch(const WgradPatch &wp, dim3 grid, size_t lds_bytes)
{
    static bool raised = false;
    if (!raised) {
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)conv_wgrad_patch_k<WM, WC, kGeo>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    hipLaunchKernelGGL((conv_wgrad_patch_k<WM, WC, kGeo>), grid, dim3(64 * 3 * WM * WC), lds_bytes, stream(), wp);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int launch_wgrad_reduce(int K, int C, int Cp, int taps, int splits, size_t out_elems, const float *partial, float *dw)
{
    // 64-channel chunks when that still leaves >= 1024 workgroups and the LDS staging stays small
    const int ch = ((size_t)K * ((C + 63) / 64) >= 1024 && taps <= 16) ? 64 : 16;
    dim3 rgrid((unsigned)K, (unsigned)((C + ch - 1) / ch));
    hipLaunchKernelGGL(wgrad_reduce_k, rgrid, dim3(256), (size_t)5 * ch * taps * sizeof(float), stream(), K, C, Cp, taps,
                       ch, splits, out_elems, partial, dw);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// What run_wgrad_patch decides before it touches memory: ok = false when the shape is not this path's
// (3x3, unit stride, pad 1; rows of 8 / 16 / 32 / 64 pixels, or 4x4 or 2x2 images).
struct WgradSetup {
    bool ok;
    WgradPatch wp;
    bool tall;            // 128 rows x 32 channels per block
    int rows;             // output channels per block: 128 (tall), 160 (x 32 channels) or 64 (x 64 channels)
    int geo, tiles, splits;
    size_t out_elems, lds_bytes;
};

WgradSetup wgrad_patch_setup(const dopt_hip_conv_desc *d, const float *dw)
{
    WgradSetup u{};
    if (d->R != 3 || d->S != 3 || d->strideH != 1 || d->strideW != 1 || d->padH != 1 || d->padW != 1) return u;
    if (d->C < 16) return u;  // a 32-channel fragment would be mostly padding
    const int W = (int)d->W, H = (int)d->H;
    WgradPatch &wp = u.wp;
    int geo;
    if (W == 8 || W == 16 || W == 32 || W == 64) {
        geo = 0;
        wp.G = 64 / W;
        if (H % wp.G != 0) return u;
        wp.bands = H / wp.G;
        wp.imgs = 1;
        wp.ppitch = W + 8;
        wp.cstride = (wp.G + 2) * wp.ppitch;
        wp.chunks_total = (int)d->N * wp.bands;
    } else if ((W == 4 && H == 4) || (W == 2 && H == 2)) {
        geo = W == 4 ? 1 : 2;
        wp.G = H;
        wp.bands = 1;
        wp.imgs = 64 / (H * W);
        if (d->N % wp.imgs != 0) return u;
        wp.ppitch = geo == 1 ? 12 : 4;
        wp.cstride = geo == 1 ? 4 * 72 : 16 * 16;
        wp.chunks_total = (int)d->N / wp.imgs;
    } else {
        return u;
    }
    while (wp.cstride % 8 != 4) wp.cstride += 4;  // 128-bit reads by 32 channels at this stride touch every LDS bank once
    // 128 rows x 32 channels, or 64 x 64 when that pads the output channels less (160 -> 192, not 256)
    // ... or 160 x 32 where that pads them less than both (160 channels: 160 rows, not 192 or 256)
    const int up64 = (int)((d->K + 63) / 64 * 64), up128 = (int)((d->K + 127) / 128 * 128), up160 = (int)((d->K + 159) / 160 * 160);
    // (by a tenth at least: 480 channels are 512 rows of the 64-row tiles, and ran no faster as 3 x 160)
    // (320 and 640 channels, which the other heights do not pad either, ran slower this way: measured)
    const bool rows160 = d->K > 64 && up160 * 11 < up64 * 10 && up160 * 11 < up128 * 10 && !no_tall_tiles();
    const bool tall = !rows160 && d->K >= 128 && up128 <= up64;
    if (!tall && !rows160 && W == 64) return u;
    const int BM = rows160 ? 160 : tall ? 128 : 64, BC = BM == 64 ? 64 : 32;
    wp.N = (int)d->N; wp.C = (int)d->C; wp.K = (int)d->K; wp.H = H; wp.W = W;
    wp.quads_row = W / 4;
    wp.mtiles = (wp.K + BM - 1) / BM;
    wp.ctiles = (wp.C + BC - 1) / BC;
    wp.dy_bytes = (size_t)wp.N * wp.K * H * W * sizeof(float);
    wp.x_bytes = (size_t)wp.N * wp.C * H * W * sizeof(float);
    const size_t out_elems = (size_t)wp.K * wp.C * 9;
    const int tiles = wp.mtiles * wp.ctiles;
    // one block per CU: never a grid slightly above the CU count (a second, nearly empty round)
    // Splits of the pixel chunks: one block per CU runs at a time, the launch takes ceil(blocks / CUs)
    // rounds of one block's duration.  Estimate (microseconds) per candidate: rounds x (chunks per
    // block x time per chunk + a fixed set-up and epilogue) + writing and re-reading the partial
    // filters; 100 tiles are better served by 5 splits (500 blocks, two nearly full rounds) than by
    // 2 (200 blocks on 256 CUs).
    int splits = 1;
    {
        const int max_by_depth = wp.chunks_total / 2 > 0 ? wp.chunks_total / 2 : 1;  // two chunks amortise the set-up
        const double t_chunk = 2.0 * BM * BC * 9 * 64 / 0.45e6;
        double best = 0.0;
        for (int sp = 1; sp <= max_by_depth && sp <= 512; sp++) {
            const int per_block = (wp.chunks_total + sp - 1) / sp;
            if (sp > 1 && (wp.chunks_total + per_block - 1) / per_block != sp) continue;
            const double rounds = (double)(((long long)tiles * sp + num_cus() - 1) / num_cus());
            double cost = rounds * (per_block * t_chunk + 8.0);
            if (sp > 1) cost += 3.0 + 2.0 * sp * out_elems * 4.0 / 4.5e6;
            if (sp == 1 || cost < best * 0.97) {
                splits = sp;
                best = cost;
            }
        }
    }
    if (out_elems % 4 != 0 || !aligned16(dw)) splits = 1;  // the split sum works on float4
    wp.chunks_per_split = (wp.chunks_total + splits - 1) / splits;
    splits = (wp.chunks_total + wp.chunks_per_split - 1) / wp.chunks_per_split;
    wp.splits = splits;
    const size_t lds_main = ((size_t)2 * BM * 68 + (size_t)2 * BC * wp.cstride + 4) * sizeof(float);
    const size_t lds_epi = (size_t)32 * (BC * 9 + 1) * sizeof(float);
    u.lds_bytes = lds_main > lds_epi ? lds_main : lds_epi;
    if (u.lds_bytes > 160 * 1024) return u;
    wp.split_stride = out_elems;
    u.tall = tall; u.rows = BM; u.geo = geo; u.tiles = tiles; u.splits = splits; u.out_elems = out_elems;
    u.ok = true;
    return u;
}

// Split lanes of the pass that adds a filter gradient's partial copies: enough blocks for small filters with
// hundreds of splits means more split lanes per block.
int wgrad_sum_lanes(size_t n4) { return n4 >= (size_t)64 * 512 ? 4 : 16; }

// out = `splits` partial copies of n4 quads added in the order `lanes` fixes (split_sum_k)
int launch_split_sum(size_t n4, int splits, int lanes, const float *partial, float *out)
{
    if (lanes == 4)
        hipLaunchKernelGGL(split_sum_k<4>, dim3((unsigned)ceil_div(n4, (size_t)64)), dim3(256), 0, stream(), n4, splits, n4,
                           (const float4 *)partial, (float4 *)out);
    else if (lanes == 16)
        hipLaunchKernelGGL(split_sum_k<16>, dim3((unsigned)ceil_div(n4, (size_t)16)), dim3(256), 0, stream(), n4, splits, n4,
                           (const float4 *)partial, (float4 *)out);
    else
        return fail(DOPT_HIP_ERR_INVALID, "split sum: %d lanes (4 or 16)", lanes);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// dw = the partial filters added in split order
int wgrad_split_sum(const WgradSetup &u, const float *partial, float *dw)
{
    const size_t n4 = u.out_elems / 4;
    return launch_split_sum(n4, u.splits, wgrad_sum_lanes(n4), partial, dw);
}

// The launch of a filled-in filter-gradient setup: tile height and pixel geometry pick the instance.
int dispatch_wgrad_patch(const WgradSetup &u)
{
    const WgradPatch &wp = u.wp;
    const dim3 grid(xcd_grid((unsigned)(u.tiles * u.splits)));
    const int geo = u.geo;
    if (u.rows == 160) return geo == 0 ? launch_wgrad_patch<5, 1, 0>(wp, grid, u.lds_bytes)
                            : geo == 1 ? launch_wgrad_patch<5, 1, 1>(wp, grid, u.lds_bytes)
                                       : launch_wgrad_patch<5, 1, 2>(wp, grid, u.lds_bytes);
    if (u.tall) return geo == 0 ? launch_wgrad_patch<4, 1, 0>(wp, grid, u.lds_bytes)
                     : geo == 1 ? launch_wgrad_patch<4, 1, 1>(wp, grid, u.lds_bytes)
                                : launch_wgrad_patch<4, 1, 2>(wp, grid, u.lds_bytes);
    return geo == 0 ? launch_wgrad_patch<2, 2, 0>(wp, grid, u.lds_bytes)
         : geo == 1 ? launch_wgrad_patch<2, 2, 1>(wp, grid, u.lds_bytes)
                    : launch_wgrad_patch<2, 2, 2>(wp, grid, u.lds_bytes);
}

int run_wgrad_patch(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw, bool *done)
{
    *done = false;
    WgradSetup u = wgrad_patch_setup(d, dw);
    if (!u.ok) return DOPT_HIP_OK;
    WgradPatch &wp = u.wp;
    float *partial = nullptr;
    if (u.splits > 1) {
        partial = (float *)workspace((size_t)u.splits * u.out_elems * sizeof(float));
        if (!partial) return DOPT_HIP_ERR_OOM;
    }
    wp.dy = dy; wp.x = x;
    wp.out = u.splits > 1 ? partial : dw;
    if (int rc = dispatch_wgrad_patch(u)) return rc;
    *done = true;
    if (u.splits > 1) return wgrad_split_sum(u, partial, dw);
    return DOPT_HIP_OK;
}

// Backward-data (on a packed filter) and filter gradient of one 3x3 layer as one launch (conv_bwd_pair_k).
// *done = false: one of the two is not a patch-kernel shape, or a combination that is not built; the
// caller runs them one after the other.  `open` as in run_patch.
template <class T, int NPMAX, int WM, int WC, int kGeo>
int launch_bwd_pair(const PatchConv &pc, const WgradPatch &wp, unsigned grid_a, unsigned grid_b, size_t lds_bytes)
{
    static bool raised = false;
    if (!raised) {
        DOPT_HIP_CHECK(hipFuncSetAttribute((const void *)conv_bwd_pair_k<T, NPMAX, WM, WC, kGeo>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    hipLaunchKernelGGL((conv_bwd_pair_k<T, NPMAX, WM, WC, kGeo>), dim3(grid_a + grid_b), dim3(768), lds_bytes, stream(), pc,
                       wp, grid_a);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}


int run_bwd_pair(const dopt_hip_conv_desc *d, size_t P, size_t Q, const float *dy, const float *prepacked, const float *x,
                 float *dx, float *dw, dopt_hip_split_sum *open, dopt_hip_split_sum *open_dw, bool *done)
{
    *done = false;
    PatchSetup a = patch_setup<true>(d, P, Q);
    WgradSetup b = wgrad_patch_setup(d, dw);
    if (!a.ok || !b.ok || !prepacked || a.pc.Cin % 16 != 0) return DOPT_HIP_OK;
    // The combinations that are built: 128 x 128 backward-data tiles on eight wavefronts, one workgroup per CU
    // (the 64 x 256 tiles of layers with up to 64 input channels run two 256-thread workgroups per CU, which a
    // launch shaped for the filter gradient's 768 threads cannot hold), with 128 x 32 filter-gradient tiles on
    // rows of 8 .. 64 pixels or on 4 x 4 images.
    // (a layer the Winograd kernel takes has its filter packed for that kernel: shape 4, not a pair)
    const int combo = a.shape == 2 && b.tall && b.geo == 0 ? 0 : a.shape == 2 && b.tall && b.geo == 1 ? 1 : -1;
    // A layer whose backward-data is the Winograd kernel on 128-row tiles: two launches, each as it would run alone, but out of ONE
    // workspace request, so that both results can stay open for the launch behind them - the filter gradient's split
    // sum rides in the batch-norm gradient there instead of being a launch of its own.  (The same for the 64-row layers
    // was measured and does not pay: they are followed by the multi-block batch norm, whose workgroups fill every CU,
    // so the riders only start when those have finished - 20 us per layer instead of the 7.6 us of the separate sum.)
    const bool two = combo < 0 && a.shape == 4 && a.BM == 128 && open_dw != nullptr && b.splits > 1;
    if (combo < 0 && !two) return DOPT_HIP_OK;
    PatchConv &pc = a.pc;
    WgradPatch &wp = b.wp;
    const int splits_a = patch_decide_splits(&a, dx);
    const size_t part_a = splits_a > 1 ? ((size_t)splits_a * pc.out_elems * sizeof(float) + 255) / 256 * 256 : 0;
    const size_t part_b = b.splits > 1 ? (size_t)b.splits * b.out_elems * sizeof(float) : 0;
    char *ws = part_a + part_b > 0 ? (char *)workspace(part_a + part_b) : nullptr;
    if (part_a + part_b > 0 && !ws) return DOPT_HIP_ERR_OOM;
    float *partial_a = (float *)ws, *partial_b = (float *)(ws + part_a);
    pc.in = dy;
    pc.wp = prepacked;
    pc.bias = nullptr;
    pc.in_bytes = (size_t)pc.N * pc.Cin * pc.IH * pc.IW * sizeof(float);
    pc.wp_bytes = a.wp_elems * sizeof(float);
    pc.out = splits_a > 1 ? partial_a : dx;
    wp.dy = dy; wp.x = x;
    wp.out = b.splits > 1 ? partial_b : dw;
    const unsigned grid_a = xcd_grid((unsigned)(a.tiles * splits_a)), grid_b = xcd_grid((unsigned)(b.tiles * b.splits));
    const size_t lds_bytes = a.lds_bytes > b.lds_bytes ? a.lds_bytes : b.lds_bytes;
    PairProbe &probe = g_pair_probe;
    const bool probing = probe.on == 1 && !capturing() && !two;
    if (probing)
        if (int rc2 = probe_begin(probe)) return rc2;
    int rc;
    if (two) {
        rc = dispatch_wgrad_patch(b);
        if (!rc) rc = dispatch_patch(a, splits_a);
    } else if (combo == 0) rc = launch_bwd_pair<GatherDeep, 16, 4, 1, 0>(pc, wp, grid_a, grid_b, lds_bytes);
    else rc = launch_bwd_pair<GatherDeep, 16, 4, 1, 1>(pc, wp, grid_a, grid_b, lds_bytes);
    if (rc) return rc;
    if (probing) {
        DOPT_HIP_CHECK(hipEventRecord(probe.events[probe.used++].second, stream()));
        const double px = (double)d->N * d->H * d->W;
        probe.flops += 2.0 * 2.0 * px * d->K * d->C * 9.0;                              // both products, every tap
        probe.bytes += 4.0 * (2.0 * px * d->C + px * d->K + 2.0 * (double)d->K * d->C * 9.0);   // dy, x, dx, filter, dw once each
    }
    *done = true;
    if (b.splits > 1 && open_dw) {   // the caller's next call adds the copies
        open_dw->partial = partial_b;
        open_dw->splits = b.splits;
        open_dw->elems = b.out_elems;
        open_dw->value = dw;
        open_dw->lanes = wgrad_sum_lanes(b.out_elems / 4);
        open_split_set(partial_b);
    } else if (b.splits > 1) {
        if (int rc2 = wgrad_split_sum(b, partial_b, dw)) return rc2;
    }
    if (splits_a > 1 && open) {   // the caller's next call adds the copies
        open->partial = partial_a;
        open->splits = splits_a;
        open->elems = pc.out_elems;
        open->C = (size_t)pc.Mout;
        open->inner = (size_t)pc.OH * pc.OW;
        open->bias = nullptr;
        open->value = dx;
        open_split_set(partial_a);
        return DOPT_HIP_OK;
    }
    if (splits_a > 1)
        return launch_splitk_reduce(pc.out_elems, splits_a, partial_a, dx, nullptr, (unsigned)pc.Mout, (unsigned)(pc.OH * pc.OW));
    return DOPT_HIP_OK;
}

using WgradSquare = Tile<128, 128, 2, 2>;
using WgradNarrow = Tile<64, 128, 1, 4>;  // K <= 64

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

int dopt_hip_conv_fwd_bias(const dopt_hip_conv_desc *d, const float *x, const float *w, const float *bias, float *y)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_fwd_bias")) return rc;
    DOPT_REQUIRE(x && w && bias && y, "dopt_hip_conv_fwd_bias: null argument");
    DOPT_ENSURE_INIT();
    return run_gather<false>(d, P, Q, x, w, y, bias);
}

int dopt_hip_conv_bwd_data(const dopt_hip_conv_desc *d, const float *dy, const float *w, float *dx)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_data")) return rc;
    DOPT_REQUIRE(dy && w && dx, "dopt_hip_conv_bwd_data: null argument");
    DOPT_ENSURE_INIT();
    return run_gather<true>(d, P, Q, dy, w, dx);
}

size_t dopt_hip_conv_packed_bytes(const dopt_hip_conv_desc *d, int bwd_data)
{
    size_t P, Q;
    if (check_desc(d, &P, &Q, "dopt_hip_conv_packed_bytes") || !ensure_init()) return 0;
    if (!bwd_data && conv_smallc_takes(d)) return 0;   // that forward kernel reads the filter as it is
    if (direct2x2_takes(d)) return d->K * d->C * 9 * sizeof(float);   // the filter as it is
    if (dense2x2_takes(d)) return dense2x2_elems(d) * sizeof(float);
    const PatchSetup u = bwd_data ? patch_setup<true>(d, P, Q) : patch_setup<false>(d, P, Q);
    // PackJob keeps strides in 32 bits
    return u.ok && d->C * 9 < (1ull << 32) ? u.wp_elems * sizeof(float) : 0;
}

int dopt_hip_conv_packed_layout(const dopt_hip_conv_desc *d, int bwd_data)
{
    if (dopt_hip_conv_packed_bytes(d, bwd_data) == 0) return -1;
    if (direct2x2_takes(d)) return 3;  // the filter itself: such kernels read [K][C][3][3], and a caller may pass the filter
    if (dense2x2_takes(d)) return 2;   // the same matrix, read transposed by backward-data
    return bwd_data ? 1 : 0;
}

int dopt_hip_conv_pack_batch(int n, const dopt_hip_conv_desc *descs, const int *bwd_data, const float *const *w,
                             float *const *packed)
{
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(n > 0 && descs && bwd_data && w && packed, "dopt_hip_conv_pack_batch: null argument");
    DOPT_ENSURE_INIT();
    PackBatch b{};
    unsigned blocks = 0;
    auto flush = [&]() -> int {
        if (b.njobs == 0) return DOPT_HIP_OK;
        hipLaunchKernelGGL(pack_batch_k, dim3(blocks), dim3(256), 0, stream(), b);
        DOPT_LAUNCH_CHECK();
        b.njobs = 0;
        blocks = 0;
        return DOPT_HIP_OK;
    };
    for (int i = 0; i < n; i++) {
        size_t P, Q;
        if (int rc = check_desc(&descs[i], &P, &Q, "dopt_hip_conv_pack_batch")) return rc;
        DOPT_REQUIRE(w[i] && packed[i] && aligned16(packed[i]), "dopt_hip_conv_pack_batch: filter %d: null or unaligned pointer", i);
        if (direct2x2_takes(&descs[i])) {   // "packed" is a plain copy (callers that know pass the filter itself instead)
            if (int rc = flush()) return rc;
            if (packed[i] != w[i])
                if (int rc = dopt_hip_copy_d2d(packed[i], w[i], descs[i].K * descs[i].C * 9 * sizeof(float))) return rc;
            continue;
        }
        if (dense2x2_takes(&descs[i]) && !(!bwd_data[i] && conv_smallc_takes(&descs[i]))) {
            if (int rc = dense2x2_pack(&descs[i], w[i], packed[i])) return rc;   // a launch of its own: the matrix is large
            continue;
        }
        const PatchSetup u = bwd_data[i] ? patch_setup<true>(&descs[i], P, Q) : patch_setup<false>(&descs[i], P, Q);
        DOPT_REQUIRE(u.ok && dopt_hip_conv_packed_bytes(&descs[i], bwd_data[i]) > 0,
                     "dopt_hip_conv_pack_batch: convolution %d does not take a packed filter", i);
        PackJob j = bwd_data[i] ? pack_job<true>(&descs[i], u, w[i], packed[i]) : pack_job<false>(&descs[i], u, w[i], packed[i]);
        j.first_block = blocks;
        blocks += j.mblocks * (unsigned)u.pc.chunks_total;
        b.job[b.njobs++] = j;
        if (b.njobs == kPackJobs)
            if (int rc = flush()) return rc;
    }
    return flush();
}

int dopt_hip_conv_fwd_bias_packed_open(const dopt_hip_conv_desc *d, const float *x, const float *packed,
                                       const float *bias, float *y, dopt_hip_split_sum *open)
{
    size_t P, Q;
    if (open) {   // complete unless the patch kernel splits below
        *open = dopt_hip_split_sum{};
        open->value = y;
    }
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_fwd_bias_packed")) return rc;
    DOPT_REQUIRE(x && packed && y, "dopt_hip_conv_fwd_bias_packed: null argument");
    DOPT_ENSURE_INIT();
    if (dopt_hip_conv_packed_layout(d, 0) == 3) {
        bool done = false;
        if (int rc = run_direct2x2<false>(d, x, packed, bias, y, &done)) return rc;
        if (done) return DOPT_HIP_OK;
        return run_dense2x2<false>(d, x, packed, nullptr, bias, y);   // operands it cannot read as quads: from the filter
    }
    if (dopt_hip_conv_packed_layout(d, 0) == 2) return run_dense2x2<false>(d, x, nullptr, packed, bias, y);
    bool done = false;
    if (int rc = run_patch<false>(d, P, Q, x, nullptr, bias, y, &done, packed, open)) return rc;
    DOPT_REQUIRE(done, "dopt_hip_conv_fwd_bias_packed: this convolution does not take a packed filter");
    return DOPT_HIP_OK;
}

int dopt_hip_conv_fwd_bias_packed(const dopt_hip_conv_desc *d, const float *x, const float *packed, const float *bias,
                                  float *y)
{
    return dopt_hip_conv_fwd_bias_packed_open(d, x, packed, bias, y, nullptr);
}

int dopt_hip_conv_bwd_data_packed_open(const dopt_hip_conv_desc *d, const float *dy, const float *packed, float *dx,
                                       dopt_hip_split_sum *open)
{
    size_t P, Q;
    if (open) {
        *open = dopt_hip_split_sum{};
        open->value = dx;
    }
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_data_packed")) return rc;
    DOPT_REQUIRE(dy && packed && dx, "dopt_hip_conv_bwd_data_packed: null argument");
    DOPT_ENSURE_INIT();
    if (dopt_hip_conv_packed_layout(d, 1) == 3) {
        bool done = false;
        if (int rc = run_direct2x2<true>(d, dy, packed, nullptr, dx, &done)) return rc;
        if (done) return DOPT_HIP_OK;
        return run_dense2x2<true>(d, dy, packed, nullptr, nullptr, dx);
    }
    if (dopt_hip_conv_packed_layout(d, 1) == 2) return run_dense2x2<true>(d, dy, nullptr, packed, nullptr, dx);
    bool done = false;
    if (int rc = run_patch<true>(d, P, Q, dy, nullptr, nullptr, dx, &done, packed, open)) return rc;
    DOPT_REQUIRE(done, "dopt_hip_conv_bwd_data_packed: this convolution does not take a packed filter");
    return DOPT_HIP_OK;
}

int dopt_hip_conv_bwd_data_packed(const dopt_hip_conv_desc *d, const float *dy, const float *packed, float *dx)
{
    return dopt_hip_conv_bwd_data_packed_open(d, dy, packed, dx, nullptr);
}

int dopt_hip_conv_bwd_pair_packed_open(const dopt_hip_conv_desc *d, const float *dy, const float *packed, const float *x,
                                       float *dx, float *dw, dopt_hip_split_sum *open, dopt_hip_split_sum *open_dw)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_pair_packed_open")) return rc;
    DOPT_REQUIRE(dy && packed && x && dx && dw, "dopt_hip_conv_bwd_pair_packed_open: null argument");
    DOPT_ENSURE_INIT();
    if (open) {
        *open = dopt_hip_split_sum{};
        open->value = dx;
    }
    if (open_dw) {
        *open_dw = dopt_hip_split_sum{};
        open_dw->value = dw;
    }
    bool done = false;
    if (int rc = run_bwd_pair(d, P, Q, dy, packed, x, dx, dw, open, open_dw, &done)) return rc;
    if (done) return DOPT_HIP_OK;
    // not a pair the one-launch kernel takes: filter gradient first (it may use the workspace), then backward-data,
    // which may leave its result open in it
    if (int rc = dopt_hip_conv_bwd_filter(d, dy, x, dw)) return rc;
    if (open) return dopt_hip_conv_bwd_data_packed_open(d, dy, packed, dx, open);
    return dopt_hip_conv_bwd_data_packed(d, dy, packed, dx);
}

int dopt_hip_conv_pair_probe(int enable)
{
    DOPT_ENSURE_INIT();
    DOPT_REQUIRE(enable >= 0 && enable <= 2, "dopt_hip_conv_pair_probe: 0 off, 1 one-launch backward pairs, 2 Winograd launches");
    g_pair_probe.on = enable;
    if (enable) {
        g_pair_probe.used = 0;
        g_pair_probe.flops = g_pair_probe.bytes = 0.0;
    }
    return DOPT_HIP_OK;
}

int dopt_hip_conv_pair_probe_read(int *launches, double *total_us, double *flops, double *bytes)
{
    DOPT_REQUIRE(launches && total_us && flops && bytes, "dopt_hip_conv_pair_probe_read: null argument");
    DOPT_ENSURE_INIT();
    PairProbe &probe = g_pair_probe;
    double us = 0.0;
    for (size_t i = 0; i < probe.used; i++) {
        DOPT_HIP_CHECK(hipEventSynchronize(probe.events[i].second));
        float ms = 0.0f;
        DOPT_HIP_CHECK(hipEventElapsedTime(&ms, probe.events[i].first, probe.events[i].second));
        us += (double)ms * 1000.0;
    }
    *launches = (int)probe.used;
    *total_us = us;
    *flops = probe.flops;
    *bytes = probe.bytes;
    return DOPT_HIP_OK;
}

int dopt_hip_split_sum_close(const dopt_hip_split_sum *open)
{
    DOPT_REQUIRE(open != nullptr, "dopt_hip_split_sum_close: null argument");
    if (open->splits == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(open->splits > 1 && open->partial && open->value && open->elems % 4 == 0 &&
                     (open->lanes > 0 || (open->C > 0 && open->inner > 0)),
                 "dopt_hip_split_sum_close: malformed description");
    DOPT_ENSURE_INIT();
    open_split_clear(open->partial);
    if (open->lanes > 0) return launch_split_sum(open->elems / 4, open->splits, open->lanes, open->partial, open->value);
    return launch_splitk_reduce(open->elems, open->splits, open->partial, open->value, open->bias, (unsigned)open->C,
                                (unsigned)open->inner);
}

int dopt_hip_conv_bwd_filter_batch(int n, const dopt_hip_conv_desc *descs, const float *const *dy, const float *const *x,
                                   float *const *dw)
{
    DOPT_REQUIRE(n >= 0 && (n == 0 || (descs && dy && x && dw)), "dopt_hip_conv_bwd_filter_batch: null argument");
    DOPT_ENSURE_INIT();
    // the filter gradients of 2x2-image layers are one dense product each, all of the same kernel: up to 8 share a launch
    int i = 0;
    while (i < n) {
        int m = 0;
        size_t C[8], K[8], N[8];
        while (i + m < n && m < 8) {
            const dopt_hip_conv_desc *d = &descs[i + m];
            size_t P, Q;
            if (check_desc(d, &P, &Q, "dopt_hip_conv_bwd_filter_batch") || !dy[i + m] || !x[i + m] || !dw[i + m] ||
                conv_smallc_takes(d) || !dense2x2_takes(d))
                break;
            C[m] = d->C; K[m] = d->K; N[m] = d->N;
            m++;
        }
        clear_error();
        int rc = DOPT_HIP_OK;
        if (m >= 2 && sgemm_fold2x2_batch(m, C, K, N, x + i, dy + i, dw + i, &rc)) {
            if (rc) return rc;
            i += m;
            continue;
        }
        if (int rc1 = dopt_hip_conv_bwd_filter(&descs[i], dy[i], x[i], dw[i])) return rc1;
        i++;
    }
    return DOPT_HIP_OK;
}

int dopt_hip_conv_bwd_filter(const dopt_hip_conv_desc *d, const float *dy, const float *x, float *dw)
{
    size_t P, Q;
    if (int rc = check_desc(d, &P, &Q, "dopt_hip_conv_bwd_filter")) return rc;
    DOPT_REQUIRE(dy && x && dw, "dopt_hip_conv_bwd_filter: null argument");
    DOPT_ENSURE_INIT();
    {
        bool done = false;
        if (int rc = conv_smallc_wgrad(d, dy, x, dw, &done)) return rc;
        if (done) return DOPT_HIP_OK;
        if (dense2x2_takes(d)) return run_dense2x2_wgrad(d, dy, x, dw);
        if (int rc = run_wgrad_patch(d, dy, x, dw, &done)) return rc;
        if (done) return DOPT_HIP_OK;
    }
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
    const int BM = big ? 128 : 64, BN = 128;
    f.mtiles = (f.K + BM - 1) / BM;
    f.ntiles = (f.ncols + BN - 1) / BN;
    const int tiles = f.mtiles * f.ntiles;
    // filter gradients are short and wide (small output, long pixel reduction): allow deep splits
    int splits = gather_splits(tiles, f.slabs_total, 2 * num_cus(), BM, BN, f.out_elems, 512);
    f.slabs_per_split = (f.slabs_total + splits - 1) / splits;
    splits = (f.slabs_total + f.slabs_per_split - 1) / f.slabs_per_split;
    f.splits = splits;
    float *partial = (float *)workspace((size_t)splits * f.out_elems * sizeof(float));
    if (!partial) return DOPT_HIP_ERR_OOM;
    f.out = partial;
    // column groups of one tile that can fall on different taps
    int gw = BN;
    while (f.Cp % gw != 0) gw /= 2;  // largest power-of-two divisor of Cp not above BN (>= 16)
    const int tpt = BN / gw;         // 1, 2, 4 or 8
    dim3 grid(xcd_grid((unsigned)(tiles * splits)));
#define DOPT_WGRAD(TILE, TPTV) hipLaunchKernelGGL((conv_wgrad_k<TILE, TPTV>), grid, dim3(TILE::THREADS), 0, stream(), f)
    if (big) {
        if (tpt == 1) DOPT_WGRAD(WgradSquare, 1);
        else if (tpt == 2) DOPT_WGRAD(WgradSquare, 2);
        else if (tpt == 4) DOPT_WGRAD(WgradSquare, 4);
        else DOPT_WGRAD(WgradSquare, 8);
    } else {
        if (tpt == 1) DOPT_WGRAD(WgradNarrow, 1);
        else if (tpt == 2) DOPT_WGRAD(WgradNarrow, 2);
        else if (tpt == 4) DOPT_WGRAD(WgradNarrow, 4);
        else DOPT_WGRAD(WgradNarrow, 8);
    }
#undef DOPT_WGRAD
    DOPT_LAUNCH_CHECK();
    return launch_wgrad_reduce(f.K, f.C, f.Cp, taps, splits, f.out_elems, partial, dw);
}

}  // extern "C"
