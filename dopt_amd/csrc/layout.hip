// Layout ops on 4-byte elements: slice, pad, repeat, rank-2 transpose.
// Replaces cuda/source/dopt/cuda/basic.d (host recursion issuing one cuMemcpy per innermost row
// for slice/pad, a per-axis byte-granular NVRTC kernel with temporaries for repeat, cublasSgeam
// for transpose) with one bandwidth-bound kernel per op.
#include "common.h"

namespace {

using namespace dopt;

constexpr int kMaxRank = 8;
constexpr int kBlock = 256;

struct NdDesc {
    int rank;
    size_t out_shape[kMaxRank];
    size_t in_shape[kMaxRank];
    size_t in_stride[kMaxRank];
    size_t offset[kMaxRank];  // slice: start, pad: before
};

unsigned grid_for(size_t n)
{
    size_t blocks = ceil_div(n, (size_t)kBlock);
    size_t cap = (size_t)num_cus() * 16;
    return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

// out[idx] = in[(coord + start) . in_stride]
__global__ __launch_bounds__(kBlock) void slice_nd(NdDesc d, size_t total, const uint32_t *in, uint32_t *out)
{
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t rem = idx, src = 0;
#pragma unroll
        for (int i = kMaxRank - 1; i >= 0; i--) {
            if (i < d.rank) {
                size_t c = rem % d.out_shape[i];
                rem /= d.out_shape[i];
                src += (c + d.offset[i]) * d.in_stride[i];
            }
        }
        out[idx] = in[src];
    }
}

// out[idx] = coord - before inside the input ? in[...] : 0   (every output element is written)
__global__ __launch_bounds__(kBlock) void pad_nd(NdDesc d, size_t total, const uint32_t *in, uint32_t *out)
{
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t rem = idx, src = 0;
        bool inside = true;
#pragma unroll
        for (int i = kMaxRank - 1; i >= 0; i--) {
            if (i < d.rank) {
                size_t c = rem % d.out_shape[i];
                rem /= d.out_shape[i];
                size_t ic = c - d.offset[i];  // wraps to a huge value when c < before
                inside = inside && (ic < d.in_shape[i]);
                src += ic * d.in_stride[i];
            }
        }
        out[idx] = inside ? in[src] : 0u;
    }
}

// out[coord] = in[coord mod in_shape]
__global__ __launch_bounds__(kBlock) void repeat_nd(NdDesc d, size_t total, const uint32_t *in, uint32_t *out)
{
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
        size_t rem = idx, src = 0;
#pragma unroll
        for (int i = kMaxRank - 1; i >= 0; i--) {
            if (i < d.rank) {
                size_t c = rem % d.out_shape[i];
                rem /= d.out_shape[i];
                src += (c % d.in_shape[i]) * d.in_stride[i];
            }
        }
        out[idx] = in[src];
    }
}

// ---- the same three maps for tensors below 2^32 elements --------------------------------------
// Coordinates are decoded with 32-bit multiply-high divisions by precomputed reciprocals, axes the
// map leaves alone are merged on the host, the outermost coordinate is the last quotient (no
// division), each lane keeps four independent loads in flight, and T is a 16-byte quad when the
// innermost axis allows it.
struct Nd32 {
    int rank;
    uint32_t out_shape[kMaxRank], out_magic[kMaxRank];
    uint32_t in_shape[kMaxRank], in_magic[kMaxRank];
    uint32_t in_stride[kMaxRank];
    uint32_t offset[kMaxRank];
};

// floor(2^32 / d) clamped to 32 bits: the quotient estimate is at most one too small
inline uint32_t recip32(uint32_t d)
{
    uint64_t m = (1ull << 32) / d;
    return m > 0xffffffffull ? 0xffffffffu : (uint32_t)m;
}

__device__ __forceinline__ void divmod32(uint32_t x, uint32_t d, uint32_t magic, uint32_t &q, uint32_t &r)
{
    q = __umulhi(x, magic);
    r = x - q * d;
    if (r >= d) {
        q++;
        r -= d;
    }
}

enum { kSlice = 0, kPad = 1, kRepeat = 2 };

template <int kMode, class T>
__global__ __launch_bounds__(kBlock) void map_nd32(Nd32 d, uint32_t total, const T *in, T *out)
{
    constexpr int U = 4;
    const uint32_t base = blockIdx.x * (uint32_t)(kBlock * U) + threadIdx.x;
    T v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t idx = base + u * kBlock;
        uint32_t rem = idx < total ? idx : 0, src = 0;   // lanes past the end decode element 0 and store nothing
        bool inside = true;
#pragma unroll
        for (int i = kMaxRank - 1; i >= 0; i--) {
            if (i >= d.rank) continue;
            uint32_t c;
            if (i > 0) divmod32(rem, d.out_shape[i], d.out_magic[i], rem, c);
            else c = rem;
            if (kMode == kSlice) c += d.offset[i];
            if (kMode == kPad) {
                c -= d.offset[i];            // wraps to a huge value left of the input
                inside = inside && c < d.in_shape[i];
            }
            if (kMode == kRepeat) {
                uint32_t q;
                divmod32(c, d.in_shape[i], d.in_magic[i], q, c);
            }
            src += c * d.in_stride[i];
        }
        // an unconditional load (element 0 stands in outside the input) keeps all four in flight
        const T got = in[inside ? src : 0];
        v[u] = inside ? got : T{};
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t idx = base + u * kBlock;
        if (idx < total) out[idx] = v[u];
    }
}

// Contiguous copy, 128-bit when both ends are 16-byte aligned.  One tile of 4 x 256 quads per block;
// a lane's four loads are all in flight before its first store.
constexpr int kCopyQuads = 4;
__global__ __launch_bounds__(kBlock) void copy_vec4(size_t n4, const uint4 *in, uint4 *out)
{
    // four named values, not an array: the compiler moved an array of quads into LDS
    const size_t i0 = (size_t)blockIdx.x * (kBlock * kCopyQuads) + threadIdx.x;
    const size_t i1 = i0 + kBlock, i2 = i0 + 2 * kBlock, i3 = i0 + 3 * kBlock;
    if (i3 < n4) {
        const uint4 a = in[i0], b = in[i1], c = in[i2], d = in[i3];
        out[i0] = a;
        out[i1] = b;
        out[i2] = c;
        out[i3] = d;
        return;
    }
    if (i0 < n4) out[i0] = in[i0];   // the ragged last tile
    if (i1 < n4) out[i1] = in[i1];
    if (i2 < n4) out[i2] = in[i2];
}

__global__ __launch_bounds__(kBlock) void copy_scalar(size_t n, const uint32_t *in, uint32_t *out)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) out[i] = in[i];
}

// [rows, cols] -> [cols, rows] through a 64x64 LDS tile (padded to 65 to stay conflict-free).
__global__ __launch_bounds__(kBlock) void transpose_tile(size_t rows, size_t cols, const uint32_t *in, uint32_t *out)
{
    __shared__ uint32_t tile[64][65];
    const size_t tiles_x = (cols + 63) / 64;
    const size_t bx = blockIdx.x % tiles_x, by = blockIdx.x / tiles_x;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
    const size_t c = bx * 64 + tx;
#pragma unroll
    for (int k = 0; k < 16; k++) {
        size_t r = by * 64 + ty + 4 * k;
        if (r < rows && c < cols) tile[ty + 4 * k][tx] = in[r * cols + c];
    }
    __syncthreads();
    const size_t orow_base = bx * 64, ocol = by * 64 + tx;  // out is [cols, rows]
#pragma unroll
    for (int k = 0; k < 16; k++) {
        size_t orow = orow_base + ty + 4 * k;
        if (orow < cols && ocol < rows) out[orow * rows + ocol] = tile[tx][ty + 4 * k];
    }
}

// The same tile moved with 128-bit accesses on both sides: rows and cols are multiples of four and both
// pointers 16-byte aligned.  Thread (r, q) of 16 x 16 reads quad q of tile row r + 16k, scatters its four
// words into the transposed tile (pitch 68 words keeps every row 16-byte aligned and spreads a
// wavefront's words over the banks), and after the barrier reads quad q of transposed row r + 16k whole.
__global__ __launch_bounds__(kBlock) void transpose_tile4(unsigned rows, unsigned cols, const uint4 *in, uint4 *out)
{
    __shared__ __attribute__((aligned(16))) uint32_t tile[64][68];
    const unsigned tiles_x = (cols + 63) / 64;
    const unsigned bx = blockIdx.x % tiles_x, by = blockIdx.x / tiles_x;
    const unsigned q = threadIdx.x & 15, r0 = threadIdx.x >> 4;
    const unsigned c = bx * 64 + 4 * q;
    uint4 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const unsigned r = by * 64 + r0 + 16 * k;
        v[k] = make_uint4(0, 0, 0, 0);
        if (r < rows && c < cols) v[k] = in[((size_t)r * cols + c) >> 2];
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const unsigned lr = r0 + 16 * k;
        tile[4 * q + 0][lr] = v[k].x;
        tile[4 * q + 1][lr] = v[k].y;
        tile[4 * q + 2][lr] = v[k].z;
        tile[4 * q + 3][lr] = v[k].w;
    }
    __syncthreads();
    const unsigned oc = by * 64 + 4 * q;   // out is [cols, rows]
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const unsigned lr = r0 + 16 * k, orow = bx * 64 + lr;
        if (orow < cols && oc < rows) out[((size_t)orow * rows + oc) >> 2] = *(const uint4 *)&tile[lr][4 * q];
    }
}

int copy_contiguous(const uint32_t *in, uint32_t *out, size_t n)
{
    if (n == 0) return DOPT_HIP_OK;
    if (aligned16(in) && aligned16(out) && n >= 4) {
        size_t n4 = n / 4;
        size_t blocks = ceil_div(n4, (size_t)kBlock * kCopyQuads);
        DOPT_REQUIRE(blocks <= 0x7fffffffu, "copy: %zu elements are more than one launch covers", n);
        hipLaunchKernelGGL(copy_vec4, dim3((unsigned)blocks), dim3(kBlock), 0, stream(), n4, (const uint4 *)in,
                           (uint4 *)out);
        DOPT_LAUNCH_CHECK();
        size_t tail = n - n4 * 4;
        if (tail) {
            hipLaunchKernelGGL(copy_scalar, dim3(1), dim3(kBlock), 0, stream(), tail, in + n4 * 4, out + n4 * 4);
            DOPT_LAUNCH_CHECK();
        }
        return DOPT_HIP_OK;
    }
    hipLaunchKernelGGL(copy_scalar, dim3(grid_for(n)), dim3(kBlock), 0, stream(), n, in, out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

size_t volume(const size_t *shape, int rank)
{
    size_t v = 1;
    for (int i = 0; i < rank; i++) v *= shape[i];
    return v;
}

void fill_strides(NdDesc &d)
{
    size_t s = 1;
    for (int i = d.rank - 1; i >= 0; i--) {
        d.in_stride[i] = s;
        s *= d.in_shape[i];
    }
}

// Runs slice / pad / repeat through map_nd32 when every extent fits 32 bits; returns -1 when it
// does not (the caller then uses the 64-bit kernels), else a status code.  The axis lists are the caller's, outermost
// first; `offset` is the slice start or the pad-before count and is ignored for repeat.
template <int kMode>
int try_map32(int rank, const size_t *in_shape, const size_t *out_shape, const size_t *offset, const void *in,
              void *out)
{
    size_t vin = 1, vout = 1;
    for (int i = 0; i < rank; i++) {
        vin *= in_shape[i];
        vout *= out_shape[i];
    }
    if (rank < 1 || vin >= (1ull << 32) || vout >= (1ull << 32) || vin == 0) return -1;
    // merge an axis into its outer neighbour when the map leaves it whole
    size_t is[kMaxRank], os[kMaxRank], of[kMaxRank];
    int r = 0;
    for (int i = 0; i < rank; i++) {
        const size_t o = kMode == kRepeat ? 0 : offset[i];
        const bool whole = in_shape[i] == out_shape[i] && o == 0;
        if (r > 0 && whole) {
            is[r - 1] *= in_shape[i];
            os[r - 1] *= out_shape[i];
            of[r - 1] *= in_shape[i];
        } else {
            is[r] = in_shape[i];
            os[r] = out_shape[i];
            of[r] = o;
            r++;
        }
    }
    // quads when the innermost axis and both pointers allow it
    const bool quads = is[r - 1] % 4 == 0 && os[r - 1] % 4 == 0 && of[r - 1] % 4 == 0 && aligned16(in) && aligned16(out);
    if (quads) {
        is[r - 1] /= 4;
        os[r - 1] /= 4;
        of[r - 1] /= 4;
        vout /= 4;
    }
    Nd32 d{};
    d.rank = r;
    uint32_t stride = 1;
    for (int i = r - 1; i >= 0; i--) {
        d.in_shape[i] = (uint32_t)is[i];
        d.out_shape[i] = (uint32_t)os[i];
        d.offset[i] = (uint32_t)of[i];
        d.in_magic[i] = recip32(d.in_shape[i]);
        d.out_magic[i] = recip32(d.out_shape[i]);
        d.in_stride[i] = stride;
        stride *= d.in_shape[i];
    }
    const unsigned blocks = (unsigned)ceil_div(vout, (size_t)kBlock * 4);
    if (quads)
        hipLaunchKernelGGL((map_nd32<kMode, uint4>), dim3(blocks), dim3(kBlock), 0, stream(), d, (uint32_t)vout,
                           (const uint4 *)in, (uint4 *)out);
    else
        hipLaunchKernelGGL((map_nd32<kMode, uint32_t>), dim3(blocks), dim3(kBlock), 0, stream(), d, (uint32_t)vout,
                           (const uint32_t *)in, (uint32_t *)out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

// ---- image augmentation: mirrored pad, crop, flips -------------------------------------------
// One lane per output pixel.  The source of output (y, x) is found backwards: undo the flips, add
// the crop offset, subtract the pad, and mirror coordinates that fall outside the image about its
// edge (edge pixel repeated, as the reference's reversed copies do).
__global__ __launch_bounds__(kBlock) void image_transform_k(uint32_t total, uint32_t C, uint32_t H, uint32_t W,
                                                            uint32_t magicW, uint32_t magicH, uint32_t magicC,
                                                            int jx, int jy, const int32_t *geom, const float *in,
                                                            float *out)
{
    const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= total) return;
    uint32_t rest, x, y, c, n;
    divmod32(idx, W, magicW, rest, x);
    divmod32(rest, H, magicH, rest, y);
    divmod32(rest, C, magicC, n, c);
    const int xoff = geom[3 * n], yoff = geom[3 * n + 1], flags = geom[3 * n + 2];
    int sx = (flags & 1) ? (int)(W - 1 - x) : (int)x;
    int sy = (flags & 2) ? (int)(H - 1 - y) : (int)y;
    sx += xoff - jx;
    sy += yoff - jy;
    sx = sx < 0 ? -sx - 1 : (sx >= (int)W ? 2 * (int)W - 1 - sx : sx);
    sy = sy < 0 ? -sy - 1 : (sy >= (int)H ? 2 * (int)H - 1 - sy : sy);
    // offsets come from device memory the host never saw: an out-of-range one must not become a stray read
    sx = sx < 0 ? 0 : (sx >= (int)W ? (int)W - 1 : sx);
    sy = sy < 0 ? 0 : (sy >= (int)H ? (int)H - 1 : sy);
    out[idx] = in[((size_t)(n * C + c) * H + sy) * W + sx];
}

// ---- many small device-to-device copies in one launch -----------------------------------------
constexpr int kBatchCopies = 48;
struct CopyBatch {  // passed by value: no table to upload
    const void *src[kBatchCopies];
    void *dst[kBatchCopies];
    unsigned words[kBatchCopies];  // 4-byte words
};

__global__ __launch_bounds__(256) void copy_batch_k(CopyBatch b)
{
    const unsigned *s = (const unsigned *)b.src[blockIdx.x];
    unsigned *d = (unsigned *)b.dst[blockIdx.x];
    const unsigned n = b.words[blockIdx.x];
    for (unsigned i = threadIdx.x; i < n; i += 256) d[i] = s[i];
}

}  // namespace

extern "C" {

int dopt_hip_slice(int rank, const size_t *in_shape, const size_t *out_shape, const size_t *start,
                   const void *in, void *out)
{
    DOPT_REQUIRE(rank >= 0 && rank <= kMaxRank, "dopt_hip_slice: rank %d not supported (max %d)", rank, kMaxRank);
    DOPT_REQUIRE(in && out && (rank == 0 || (in_shape && out_shape && start)), "dopt_hip_slice: null argument");
    for (int i = 0; i < rank; i++)
        DOPT_REQUIRE(start[i] + out_shape[i] <= in_shape[i] && out_shape[i] > 0,
                     "dopt_hip_slice: axis %d: [%zu, %zu) outside extent %zu", i, start[i], start[i] + out_shape[i],
                     in_shape[i]);
    DOPT_ENSURE_INIT();
    size_t total = volume(out_shape, rank);
    // A slice that only cuts the outermost axis (BN's rank-1 unpacking, row blocks) is one
    // contiguous run.
    bool contiguous = true;
    for (int i = 1; i < rank; i++) contiguous = contiguous && start[i] == 0 && out_shape[i] == in_shape[i];
    if (contiguous) {
        size_t inner = rank > 0 ? volume(in_shape + 1, rank - 1) : 1;
        size_t off = rank > 0 ? start[0] * inner : 0;
        return copy_contiguous((const uint32_t *)in + off, (uint32_t *)out, total);
    }
    if (int rc = try_map32<kSlice>(rank, in_shape, out_shape, start, in, out); rc >= 0) return rc;
    NdDesc d{};
    d.rank = rank;
    for (int i = 0; i < rank; i++) {
        d.out_shape[i] = out_shape[i];
        d.in_shape[i] = in_shape[i];
        d.offset[i] = start[i];
    }
    fill_strides(d);
    hipLaunchKernelGGL(slice_nd, dim3(grid_for(total)), dim3(kBlock), 0, stream(), d, total, (const uint32_t *)in,
                       (uint32_t *)out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_pad(int rank, const size_t *in_shape, const size_t *out_shape, const size_t *before,
                 const void *in, void *out)
{
    DOPT_REQUIRE(rank >= 0 && rank <= kMaxRank, "dopt_hip_pad: rank %d not supported (max %d)", rank, kMaxRank);
    DOPT_REQUIRE(rank == 0 || (in_shape && out_shape && before), "dopt_hip_pad: null argument");
    for (int i = 0; i < rank; i++)
        DOPT_REQUIRE(before[i] + in_shape[i] <= out_shape[i], "dopt_hip_pad: axis %d: input does not fit the output", i);
    size_t total = volume(out_shape, rank);
    if (total == 0) return DOPT_HIP_OK;
    // (an empty input has no buffer: the result is all padding)
    DOPT_REQUIRE(out && (in || volume(in_shape, rank) == 0), "dopt_hip_pad: null argument");
    DOPT_ENSURE_INIT();
    if (rank == 0) return copy_contiguous((const uint32_t *)in, (uint32_t *)out, 1);
    if (int rc = try_map32<kPad>(rank, in_shape, out_shape, before, in, out); rc >= 0) return rc;
    NdDesc d{};
    d.rank = rank;
    for (int i = 0; i < rank; i++) {
        d.out_shape[i] = out_shape[i];
        d.in_shape[i] = in_shape[i];
        d.offset[i] = before[i];
    }
    fill_strides(d);
    hipLaunchKernelGGL(pad_nd, dim3(grid_for(total)), dim3(kBlock), 0, stream(), d, total, (const uint32_t *)in,
                       (uint32_t *)out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_repeat(int rank, const size_t *in_shape, const size_t *reps, const void *in, void *out)
{
    DOPT_REQUIRE(rank >= 0 && rank <= kMaxRank, "dopt_hip_repeat: rank %d not supported (max %d)", rank, kMaxRank);
    DOPT_REQUIRE(rank == 0 || (in_shape && reps), "dopt_hip_repeat: null argument");
    DOPT_REQUIRE((in && out) || volume(in_shape, rank) == 0, "dopt_hip_repeat: null argument");   // an empty tensor has no buffer
    DOPT_ENSURE_INIT();
    NdDesc d{};
    d.rank = rank;
    bool identity = true;
    for (int i = 0; i < rank; i++) {
        DOPT_REQUIRE(reps[i] > 0, "dopt_hip_repeat: repetitions must be positive");
        d.in_shape[i] = in_shape[i];
        d.out_shape[i] = in_shape[i] * reps[i];
        identity = identity && reps[i] == 1;
    }
    size_t total = volume(d.out_shape, rank);
    if (total == 0) return DOPT_HIP_OK;
    if (identity) return copy_contiguous((const uint32_t *)in, (uint32_t *)out, total);  // cuda/basic.d:168-172
    if (int rc = try_map32<kRepeat>(rank, d.in_shape, d.out_shape, nullptr, in, out); rc >= 0) return rc;
    fill_strides(d);
    hipLaunchKernelGGL(repeat_nd, dim3(grid_for(total)), dim3(kBlock), 0, stream(), d, total, (const uint32_t *)in,
                       (uint32_t *)out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_image_transform(size_t N, size_t C, size_t H, size_t W, size_t jitterX, size_t jitterY,
                             const int32_t *geom, const float *in, float *out)
{
    const size_t total = N * C * H * W;
    if (total == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(geom && in && out, "dopt_hip_image_transform: null argument");
    DOPT_REQUIRE(in != out, "dopt_hip_image_transform: the batch cannot be transformed in place");
    DOPT_REQUIRE(total < (1ull << 32), "dopt_hip_image_transform: batch of %zu values is too large", total);
    // one mirror image per side: the pad cannot be wider than the image it mirrors
    DOPT_REQUIRE(jitterX <= W && jitterY <= H, "dopt_hip_image_transform: jitter (%zu, %zu) exceeds the image (%zu, %zu)",
                 jitterX, jitterY, W, H);
    DOPT_ENSURE_INIT();
    hipLaunchKernelGGL(image_transform_k, dim3((unsigned)ceil_div(total, (size_t)kBlock)), dim3(kBlock), 0, stream(),
                       (uint32_t)total, (uint32_t)C, (uint32_t)H, (uint32_t)W, recip32((uint32_t)W),
                       recip32((uint32_t)H), recip32((uint32_t)C), (int)jitterX, (int)jitterY, geom, in, out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_transpose2d(size_t rows, size_t cols, const void *in, void *out)
{
    if (rows * cols == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(in && out, "dopt_hip_transpose2d: null argument");
    DOPT_ENSURE_INIT();
    if (rows == 1 || cols == 1) return copy_contiguous((const uint32_t *)in, (uint32_t *)out, rows * cols);
    size_t tiles = ceil_div(cols, 64) * ceil_div(rows, 64);
    DOPT_REQUIRE(tiles <= 0x7fffffffu, "dopt_hip_transpose2d: matrix too large");
    if ((rows & 3) == 0 && (cols & 3) == 0 && aligned16(in) && aligned16(out) && rows < (1u << 31) && cols < (1u << 31)) {
        hipLaunchKernelGGL(transpose_tile4, dim3((unsigned)tiles), dim3(kBlock), 0, stream(), (unsigned)rows, (unsigned)cols,
                           (const uint4 *)in, (uint4 *)out);
        DOPT_LAUNCH_CHECK();
        return DOPT_HIP_OK;
    }
    hipLaunchKernelGGL(transpose_tile, dim3((unsigned)tiles), dim3(kBlock), 0, stream(), rows, cols,
                       (const uint32_t *)in, (uint32_t *)out);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

int dopt_hip_copy_d2d_batch(int n, void *const *dst, const void *const *src, const size_t *bytes)
{
    DOPT_REQUIRE(n == 0 || (dst && src && bytes), "dopt_hip_copy_d2d_batch: null argument");
    DOPT_ENSURE_INIT();
    CopyBatch b;
    int filled = 0;
    auto flush = [&]() -> int {
        if (filled == 0) return DOPT_HIP_OK;
        hipLaunchKernelGGL(copy_batch_k, dim3((unsigned)filled), dim3(256), 0, stream(), b);
        DOPT_LAUNCH_CHECK();
        filled = 0;
        return DOPT_HIP_OK;
    };
    for (int i = 0; i < n; i++) {
        if (bytes[i] == 0) continue;
        DOPT_REQUIRE(dst[i] && src[i], "dopt_hip_copy_d2d_batch: null pointer");
        const bool small = bytes[i] <= 65536 && bytes[i] % 4 == 0 &&
                           (reinterpret_cast<uintptr_t>(dst[i]) & 3u) == 0 && (reinterpret_cast<uintptr_t>(src[i]) & 3u) == 0;
        if (!small) {
            // the copies are sequential: what is still waiting in the batch goes first
            if (int rc = flush()) return rc;
            if (int rc = dopt_hip_copy_d2d(dst[i], src[i], bytes[i])) return rc;
            continue;
        }
        // copies of one launch run side by side: a copy that reads or rewrites what an earlier one
        // of the batch writes, or that writes what an earlier one reads, starts a new launch
        for (int j = 0; j < filled; j++) {
            const size_t len = (size_t)b.words[j] * 4;
            const char *d0 = (const char *)b.dst[j], *d1 = d0 + len;
            const char *r0 = (const char *)b.src[j], *r1 = r0 + len;
            const char *s0 = (const char *)src[i], *t0 = (const char *)dst[i];
            if ((s0 < d1 && s0 + bytes[i] > d0) || (t0 < d1 && t0 + bytes[i] > d0) || (t0 < r1 && t0 + bytes[i] > r0)) {
                if (int rc = flush()) return rc;
                break;
            }
        }
        b.src[filled] = src[i];
        b.dst[filled] = dst[i];
        b.words[filled] = (unsigned)(bytes[i] / 4);
        if (++filled == kBatchCopies)
            if (int rc = flush()) return rc;
    }
    return flush();
}

}  // extern "C"
