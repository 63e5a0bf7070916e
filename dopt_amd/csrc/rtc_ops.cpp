// Pointwise and reduction ops: gfx950 HIP source templates instantiated per (op, dtype) through
// hipRTC.  Replaces the NVRTC string generator of cuda/source/dopt/cuda/math.d:129-205 (one
// scalar element per thread, device sync after each launch) with 128-bit vector loads, four
// independent loads in flight per lane and no host synchronisation.  Semantics follow the CPU
// evaluator, cpu/source/dopt/cpu/math.d:312-437 (pointwise), :90-247 (sum / maxElement) and
// :249-310 (argmin).
#include <cstring>
#include <string>
#include <vector>

#include "common.h"
#include "pw_ops.h"
#include <limits>

namespace {

using namespace dopt;

struct OpInfo {
    const char *name;
    int arity;
    const char *expr_f32;
    const char *expr_i32;
};

// `a`, `b` are the operands of type T; the table is pw_ops.h, each expression as the text the run-time compiler gets.
const OpInfo kOps[] = {
#define DOPT_PW_ROW(name, arity, f32, i32) {#name, arity, #f32, #i32},
    DOPT_PW_OPS(DOPT_PW_ROW)
#undef DOPT_PW_ROW
};

const OpInfo *find_op(const char *name)
{
    for (const OpInfo &o : kOps)
        if (!strcmp(o.name, name)) return &o;
    return nullptr;
}

const char *kPointwiseBody = R"SRC(
typedef T T4 __attribute__((ext_vector_type(4)));
#define UNROLL 4
#define BLOCK 256

// std.math.pow(int, int): exponentiation by squaring with wrapping multiplies.
__device__ inline int dopt_ipow(int x, int n)
{
    if (n < 0) {
        if (x == 1) return 1;
        if (x == -1) return (n & 1) ? -1 : 1;
        return 0;
    }
    unsigned p = 1u, v = (unsigned)x, m = (unsigned)n;
    while (m) {
        if (m & 1u) p *= v;
        m >>= 1;
        v *= v;
    }
    return (int)p;
}

__device__ inline T dopt_op(T a, T b) { return (T)(OPEXPR); }

// 16-byte aligned operands: each lane keeps UNROLL independent 128-bit loads per operand in flight.
extern "C" __global__ __launch_bounds__(BLOCK) void pw_vec(size_t n, const T *a, const T *b, T *o)
{
    const size_t n4 = n >> 2;
    const T4 *a4 = (const T4 *)a;
    const T4 *b4 = (const T4 *)b;
    T4 *o4 = (T4 *)o;
    for (size_t base = (size_t)blockIdx.x * (BLOCK * UNROLL); base < n4;
         base += (size_t)gridDim.x * (BLOCK * UNROLL)) {
        T4 x[UNROLL], y[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            size_t i = base + (size_t)u * BLOCK + threadIdx.x;
            if (i < n4) {
                x[u] = a4[i];
#if ARITY == 2
                y[u] = b4[i];
#else
                y[u] = x[u];
#endif
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            size_t i = base + (size_t)u * BLOCK + threadIdx.x;
            if (i < n4) {
                T4 r;
                r.x = dopt_op(x[u].x, y[u].x);
                r.y = dopt_op(x[u].y, y[u].y);
                r.z = dopt_op(x[u].z, y[u].z);
                r.w = dopt_op(x[u].w, y[u].w);
                o4[i] = r;
            }
        }
    }
    if (blockIdx.x == 0) {
        size_t i = (n4 << 2) + threadIdx.x;
        if (i < n) {
#if ARITY == 2
            o[i] = dopt_op(a[i], b[i]);
#else
            o[i] = dopt_op(a[i], a[i]);
#endif
        }
    }
}

// Any alignment.
extern "C" __global__ __launch_bounds__(BLOCK) void pw_scalar(size_t n, const T *a, const T *b, T *o)
{
    for (size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (size_t)gridDim.x * BLOCK) {
#if ARITY == 2
        o[i] = dopt_op(a[i], b[i]);
#else
        o[i] = dopt_op(a[i], a[i]);
#endif
    }
}
)SRC";

std::string pointwise_source(const OpInfo &op, int dtype)
{
    std::string s;
    s += dtype == DOPT_HIP_F32 ? "typedef float T;\n" : "typedef int T;\n";
    s += "#define ARITY " + std::to_string(op.arity) + "\n";
    s += std::string("#define OPEXPR ") + (dtype == DOPT_HIP_F32 ? op.expr_f32 : op.expr_i32) + "\n";
    s += kPointwiseBody;
    return s;
}

// ------------------------------------------------------------------------------ pointwise chains
// A DAG of pointwise nodes over equally long operands as ONE kernel: every node keeps its own
// function (the same expression the stand-alone kernel of that op evaluates, compiled without
// contraction), intermediate values stay in fp32 registers, so the result equals running the
// nodes one kernel at a time bit for bit.  Operand k < nin is input k (a vector, or a one-element
// tensor broadcast to every position); operand nin + j is node j.  Outputs: the last node.
std::string chain_source(int dtype, int nin, const unsigned char *kind, int nnodes, const OpInfo *const *ops,
                         const int *lhs, const int *rhs)
{
    // kind: 0 an n-element tensor; 1 one element, read at every position; 2 one element per row of the
    // [n / inner, inner] view (index e / inner); 3 one element per column (index e % inner)
    bool grid = false;
    for (int k = 0; k < nin; k++) grid = grid || kind[k] >= 2;
    std::string s = dtype == DOPT_HIP_F32 ? "typedef float T;\n" : "typedef int T;\n";
    s += "typedef T T4 __attribute__((ext_vector_type(4)));\n#define BLOCK 256\n";
    s += R"SRC(
__device__ inline int dopt_ipow(int x, int n)
{
    if (n < 0) {
        if (x == 1) return 1;
        if (x == -1) return (n & 1) ? -1 : 1;
        return 0;
    }
    unsigned p = 1u, v = (unsigned)x, m = (unsigned)n;
    while (m) {
        if (m & 1u) p *= v;
        m >>= 1;
        v *= v;
    }
    return (int)p;
}
)SRC";
    for (int j = 0; j < nnodes; j++)
        s += "__device__ inline T f" + std::to_string(j) + "(T a, T b) { return (T)(" +
             (dtype == DOPT_HIP_F32 ? ops[j]->expr_f32 : ops[j]->expr_i32) + "); }\n";
    // `lane` is a component suffix of the quads (".x") or "" in the one-element-at-a-time code
    auto operand = [&](int k, const char *lane) -> std::string {
        if (k >= nin) return "t" + std::to_string(k - nin);
        if (kind[k] == 1) return "s" + std::to_string(k);
        if (kind[k] == 2) return "r" + std::to_string(k);
        return "x" + std::to_string(k) + lane;
    };
    auto body = [&](const char *lane, const std::string &dst) {
        std::string b = "        {\n";
        for (int j = 0; j < nnodes; j++) {
            const std::string a = operand(lhs[j], lane), c = ops[j]->arity == 2 ? operand(rhs[j], lane) : a;
            b += "            const T t" + std::to_string(j) + " = f" + std::to_string(j) + "(" + a + ", " + c + ");\n";
        }
        b += "            " + dst + " = t" + std::to_string(nnodes - 1) + ";\n        }\n";
        return b;
    };
    std::string params = "size_t n, size_t inner";
    for (int k = 0; k < nin; k++) params += ", const T *i" + std::to_string(k);
    params += ", T *o";
    std::string scalars;
    for (int k = 0; k < nin; k++)
        if (kind[k] == 1) scalars += "    const T s" + std::to_string(k) + " = i" + std::to_string(k) + "[0];\n";

    // quads (inner is a multiple of four whenever rows or columns are indexed, so a quad never
    // straddles a row): one quad per lane and pass, all loads before the first use
    s += "extern \"C\" __global__ __launch_bounds__(BLOCK) void chain_vec(" + params + ")\n{\n" + scalars;
    s += "    const size_t n4 = n >> 2, inner4 = inner >> 2;\n";
    s += "    for (size_t q = (size_t)blockIdx.x * BLOCK + threadIdx.x; q < n4; q += (size_t)gridDim.x * BLOCK) {\n";
    if (grid) s += "        const size_t row = q / inner4, colq = q - row * inner4;\n";
    for (int k = 0; k < nin; k++) {
        const std::string i = std::to_string(k);
        if (kind[k] == 0) s += "        const T4 x" + i + " = ((const T4 *)i" + i + ")[q];\n";
        if (kind[k] == 2) s += "        const T r" + i + " = i" + i + "[row];\n";
        if (kind[k] == 3) s += "        const T4 x" + i + " = ((const T4 *)i" + i + ")[colq];\n";
    }
    s += "        T4 r;\n";
    for (const char *lane : {".x", ".y", ".z", ".w"}) s += body(lane, std::string("r") + lane);
    s += "        ((T4 *)o)[q] = r;\n    }\n";
    // the last n % 4 elements (none when rows or columns are indexed)
    s += "    if (blockIdx.x == 0) {\n        const size_t e = (n4 << 2) + threadIdx.x;\n        if (e < n) {\n";
    if (grid) s += "            const size_t row = e / inner, col = e - row * inner;\n";
    for (int k = 0; k < nin; k++) {
        const std::string i = std::to_string(k);
        if (kind[k] == 0) s += "            const T x" + i + " = i" + i + "[e];\n";
        if (kind[k] == 2) s += "            const T r" + i + " = i" + i + "[row];\n";
        if (kind[k] == 3) s += "            const T x" + i + " = i" + i + "[col];\n";
    }
    s += body("", "o[e]");
    s += "        }\n    }\n}\n";

    s += "extern \"C\" __global__ __launch_bounds__(BLOCK) void chain_scalar(" + params + ")\n{\n" + scalars;
    s += "    for (size_t e = (size_t)blockIdx.x * BLOCK + threadIdx.x; e < n; e += (size_t)gridDim.x * BLOCK) {\n";
    if (grid) s += "        const size_t row = e / inner, col = e - row * inner;\n";
    for (int k = 0; k < nin; k++) {
        const std::string i = std::to_string(k);
        if (kind[k] == 0) s += "        const T x" + i + " = i" + i + "[e];\n";
        if (kind[k] == 2) s += "        const T r" + i + " = i" + i + "[row];\n";
        if (kind[k] == 3) s += "        const T x" + i + " = i" + i + "[col];\n";
    }
    s += body("", "o[e]");
    s += "    }\n}\n";
    return s;
}

// ------------------------------------------------------------------------------ reductions

const char *kReduceBody = R"SRC(
#define BLOCK 256

__device__ inline T combine(T a, T b) { return (T)(COMBINE); }

// what is folded is PRE(element): the element itself, or its square rounded to T (the value mul(x, x) would have stored)
__device__ inline T4 pre4(T4 v)
{
    T4 r;
    r.x = PRE(v.x); r.y = PRE(v.y); r.z = PRE(v.z); r.w = PRE(v.w);
    return r;
}

__device__ inline T wave_reduce(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T o = __shfl_down(v, off, 64);
        v = combine(v, o);
    }
    return v;
}

__device__ inline T block_reduce(T v)
{
    __shared__ T part[BLOCK / 64];
    v = wave_reduce(v);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < BLOCK / 64; w++) v = combine(v, part[w]);
    }
    return v;  // valid in thread 0
}

// Contiguous rows: block (row o, chunk c) reduces in[o*R + c*chunk ... ) into out[o*nchunks + c].
extern "C" __global__ __launch_bounds__(BLOCK) void red_rows(const T *in, T *out, size_t R, size_t chunk,
                                                              size_t nchunks)
{
    const size_t o = blockIdx.x / nchunks, c = blockIdx.x % nchunks;
    const size_t start = c * chunk;
    size_t end = start + chunk;
    if (end > R) end = R;
    const T *row = in + o * R;
    T acc0 = (T)(IDENT), acc1 = (T)(IDENT), acc2 = (T)(IDENT), acc3 = (T)(IDENT);
    size_t i = start + threadIdx.x;
    for (; i + 3 * BLOCK < end; i += 4 * BLOCK) {
        T v0 = PRE(row[i]), v1 = PRE(row[i + BLOCK]), v2 = PRE(row[i + 2 * BLOCK]), v3 = PRE(row[i + 3 * BLOCK]);
        acc0 = combine(acc0, v0);
        acc1 = combine(acc1, v1);
        acc2 = combine(acc2, v2);
        acc3 = combine(acc3, v3);
    }
    for (; i < end; i += BLOCK) acc0 = combine(acc0, PRE(row[i]));
    T acc = combine(combine(acc0, acc1), combine(acc2, acc3));
    acc = block_reduce(acc);
    if (threadIdx.x == 0) out[blockIdx.x] = acc;
}

// The same with 128-bit loads: R and chunk are multiples of 4 and `in` is 16-byte aligned.
extern "C" __global__ __launch_bounds__(BLOCK) void red_rows4(const T *in, T *out, size_t R, size_t chunk,
                                                               size_t nchunks)
{
    const size_t o = blockIdx.x / nchunks, c = blockIdx.x % nchunks;
    const size_t start = c * chunk;
    size_t end = start + chunk;
    if (end > R) end = R;
    const T4 *row = (const T4 *)(in + o * R);
    const size_t q0 = start / 4, q1 = end / 4;
    T acc0 = (T)(IDENT), acc1 = (T)(IDENT), acc2 = (T)(IDENT), acc3 = (T)(IDENT);
    size_t i = q0 + threadIdx.x;
    for (; i + 3 * BLOCK < q1; i += 4 * BLOCK) {
        T4 v0 = pre4(row[i]), v1 = pre4(row[i + BLOCK]), v2 = pre4(row[i + 2 * BLOCK]), v3 = pre4(row[i + 3 * BLOCK]);
        acc0 = combine(acc0, combine(combine(v0.x, v0.y), combine(v0.z, v0.w)));
        acc1 = combine(acc1, combine(combine(v1.x, v1.y), combine(v1.z, v1.w)));
        acc2 = combine(acc2, combine(combine(v2.x, v2.y), combine(v2.z, v2.w)));
        acc3 = combine(acc3, combine(combine(v3.x, v3.y), combine(v3.z, v3.w)));
    }
    for (; i < q1; i += BLOCK) {
        T4 v0 = pre4(row[i]);
        acc0 = combine(acc0, combine(combine(v0.x, v0.y), combine(v0.z, v0.w)));
    }
    T acc = combine(combine(acc0, acc1), combine(acc2, acc3));
    acc = block_reduce(acc);
    if (threadIdx.x == 0) out[blockIdx.x] = acc;
}

// The same order of sums from a buffer that is not 16-byte aligned (a view into a larger tensor): four 32-bit loads
// per quad, so that a value does not depend on where its operand happens to start.
__device__ inline T4 ld4(const T *p)
{
    T4 r;
    r.x = PRE(p[0]); r.y = PRE(p[1]); r.z = PRE(p[2]); r.w = PRE(p[3]);
    return r;
}
extern "C" __global__ __launch_bounds__(BLOCK) void red_rows4u(const T *in, T *out, size_t R, size_t chunk,
                                                                size_t nchunks)
{
    const size_t o = blockIdx.x / nchunks, c = blockIdx.x % nchunks;
    const size_t start = c * chunk;
    size_t end = start + chunk;
    if (end > R) end = R;
    const T *row = in + o * R;
    const size_t q0 = start / 4, q1 = end / 4;
    T acc0 = (T)(IDENT), acc1 = (T)(IDENT), acc2 = (T)(IDENT), acc3 = (T)(IDENT);
    size_t i = q0 + threadIdx.x;
    for (; i + 3 * BLOCK < q1; i += 4 * BLOCK) {
        T4 v0 = ld4(row + 4 * i), v1 = ld4(row + 4 * (i + BLOCK)), v2 = ld4(row + 4 * (i + 2 * BLOCK)), v3 = ld4(row + 4 * (i + 3 * BLOCK));
        acc0 = combine(acc0, combine(combine(v0.x, v0.y), combine(v0.z, v0.w)));
        acc1 = combine(acc1, combine(combine(v1.x, v1.y), combine(v1.z, v1.w)));
        acc2 = combine(acc2, combine(combine(v2.x, v2.y), combine(v2.z, v2.w)));
        acc3 = combine(acc3, combine(combine(v3.x, v3.y), combine(v3.z, v3.w)));
    }
    for (; i < q1; i += BLOCK) {
        T4 v0 = ld4(row + 4 * i);
        acc0 = combine(acc0, combine(combine(v0.x, v0.y), combine(v0.z, v0.w)));
    }
    T acc = combine(combine(acc0, acc1), combine(acc2, acc3));
    acc = block_reduce(acc);
    if (threadIdx.x == 0) out[blockIdx.x] = acc;
}

// Strided lanes: thread (o, j) folds in[(o*R + r)*inner + j] over r in ascending r (the order of
// the reference's vector adds), coalesced across j.  Eight loads are in flight per lane; the
// adds stay sequential.
extern "C" __global__ __launch_bounds__(BLOCK) void red_cols(const T *in, T *out, size_t outer, size_t R,
                                                              size_t inner)
{
    const size_t total = outer * inner;
    for (size_t idx = (size_t)blockIdx.x * BLOCK + threadIdx.x; idx < total; idx += (size_t)gridDim.x * BLOCK) {
        const size_t o = idx / inner, j = idx % inner;
        const T *p = in + o * R * inner + j;
        T acc = (T)(IDENT);
        size_t r = 0;
        for (; r + 8 <= R; r += 8) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = PRE(p[(r + u) * inner]);
#pragma unroll
            for (int u = 0; u < 8; u++) acc = combine(acc, v[u]);
        }
        for (; r < R; r++) acc = combine(acc, PRE(p[r * inner]));
        out[idx] = acc;
    }
}
)SRC";

const char *kArgminBody = R"SRC(
#define BLOCK 256
// Thread (o, j) scans the axis with a strict '<' against the type's maximum: the first minimum
// wins and a lane that never fires keeps index 0 (cpu/math.d:281-296).
extern "C" __global__ __launch_bounds__(BLOCK) void argmin_k(const T *in, int *out, size_t outer, size_t A,
                                                              size_t vol)
{
    const size_t total = outer * vol;
    for (size_t idx = (size_t)blockIdx.x * BLOCK + threadIdx.x; idx < total; idx += (size_t)gridDim.x * BLOCK) {
        const size_t o = idx / vol, j = idx % vol;
        const T *p = in + o * A * vol + j;
        T best = (T)(TMAX);
        int bi = 0;
        for (size_t i = 0; i < A; i++) {
            T v = p[i * vol];
            if (v < best) {
                best = v;
                bi = (int)i;
            }
        }
        out[idx] = bi;
    }
}

// Innermost axis (vol == 1): one wavefront per row, lanes stride along the row.  Each lane keeps
// the first minimum of its own elements; lanes are then merged preferring the smaller value and,
// on equal values, the smaller index -- the first minimum of the row, as the scan above finds it.
extern "C" __global__ __launch_bounds__(BLOCK) void argmin_rows_k(const T *in, int *out, size_t rows, size_t A)
{
    const size_t row = (size_t)blockIdx.x * (BLOCK / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const T *p = in + row * A;
    T best = (T)(TMAX);
    int bi = 0x7fffffff;  // "never fired"
    size_t i = lane;
    for (; i + 192 < A; i += 256) {   // four loads in flight; tested in index order
        T v0 = p[i], v1 = p[i + 64], v2 = p[i + 128], v3 = p[i + 192];
        if (v0 < best) { best = v0; bi = (int)i; }
        if (v1 < best) { best = v1; bi = (int)(i + 64); }
        if (v2 < best) { best = v2; bi = (int)(i + 128); }
        if (v3 < best) { best = v3; bi = (int)(i + 192); }
    }
    for (; i < A; i += 64) {
        T v = p[i];
        if (v < best) {
            best = v;
            bi = (int)i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T ov = __shfl_down(best, off, 64);
        int oi = __shfl_down(bi, off, 64);
        if (ov < best || (ov == best && oi < bi)) {
            best = ov;
            bi = oi;
        }
    }
    if (lane == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}

// The same with 128-bit loads (A a multiple of four, 16-byte aligned rows): a lane's elements still
// come in ascending index order, so its first minimum is found the same way.
extern "C" __global__ __launch_bounds__(BLOCK) void argmin_rows4_k(const T *in, int *out, size_t rows, size_t A)
{
    const size_t row = (size_t)blockIdx.x * (BLOCK / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const T4 *p = (const T4 *)(in + row * A);
    const size_t A4 = A / 4;
    T best = (T)(TMAX);
    int bi = 0x7fffffff;
#define TEST4(v, q)                                              \
    if (v.x < best) { best = v.x; bi = (int)(4 * (q)); }         \
    if (v.y < best) { best = v.y; bi = (int)(4 * (q) + 1); }     \
    if (v.z < best) { best = v.z; bi = (int)(4 * (q) + 2); }     \
    if (v.w < best) { best = v.w; bi = (int)(4 * (q) + 3); }
    size_t i = lane;
    for (; i + 192 < A4; i += 256) {
        T4 v0 = p[i], v1 = p[i + 64], v2 = p[i + 128], v3 = p[i + 192];
        TEST4(v0, i) TEST4(v1, i + 64) TEST4(v2, i + 128) TEST4(v3, i + 192)
    }
    for (; i < A4; i += 64) {
        T4 v = p[i];
        TEST4(v, i)
    }
#undef TEST4
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T ov = __shfl_down(best, off, 64);
        int oi = __shfl_down(bi, off, 64);
        if (ov < best || (ov == best && oi < bi)) {
            best = ov;
            bi = oi;
        }
    }
    if (lane == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}
)SRC";

std::string reduce_source(bool is_sum, int dtype, bool square = false)
{
    std::string s;
    bool f = dtype == DOPT_HIP_F32;
    s += f ? "typedef float T;\ntypedef float4 T4;\n" : "typedef int T;\ntypedef int4 T4;\n";
    if (is_sum) {
        s += f ? "#define COMBINE a + b\n" : "#define COMBINE (int)((unsigned)a + (unsigned)b)\n";
        s += "#define IDENT 0\n";
    } else {
        // The reference folds max(acc, element) = acc < element ? element : acc from -T.max, which passes over a NaN
        // element (cpu/math.d:183-187).  Here elements also meet each other first (the four of a 128-bit load, the
        // lanes of a wavefront), so a NaN on the left has to give way as well, or it would hide its partners.
        s += "#define COMBINE (a < b || a != a ? b : a)\n";
        // identity -T.max (cpu/math.d:186): int32 starts at -INT_MAX, not INT_MIN
        s += f ? "#define IDENT -3.402823466e+38f\n" : "#define IDENT -2147483647\n";
    }
    s += square ? "#define PRE(v) ((T)((v) * (v)))\n" : "#define PRE(v) (v)\n";
    s += kReduceBody;
    return s;
}

std::string argmin_source(int dtype)
{
    std::string s;
    s += dtype == DOPT_HIP_F32 ? "typedef float T;\ntypedef float4 T4;\n#define TMAX 3.402823466e+38f\n"
                               : "typedef int T;\ntypedef int4 T4;\n#define TMAX 2147483647\n";
    s += kArgminBody;
    return s;
}

unsigned grid_for(size_t work_items_per_block_unit, size_t units)
{
    size_t blocks = ceil_div(units, work_items_per_block_unit);
    size_t cap = (size_t)num_cus() * 8;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (unsigned)blocks;
}

int check_dtype(int dtype)
{
    if (dtype != DOPT_HIP_F32 && dtype != DOPT_HIP_I32)
        return fail(DOPT_HIP_ERR_UNSUPPORTED, "Element type not supported.");
    return DOPT_HIP_OK;
}

// One (outer, R, inner) reduction pass on the device.
// `rows_plain` adds the partial results of a split row: the first stage may fold PRE(element), the second never does.
struct ReduceKernels {
    hipFunction_t rows, rows4, rows4u, cols;
};
int reduce_kernels(const std::string &key, const std::string &src, ReduceKernels *k)
{
    if (int rc = rtc_get(key + ":rows", src, "red_rows", &k->rows)) return rc;
    if (int rc = rtc_get(key + ":rows4", src, "red_rows4", &k->rows4)) return rc;
    if (int rc = rtc_get(key + ":rows4u", src, "red_rows4u", &k->rows4u)) return rc;
    return rtc_get(key + ":cols", src, "red_cols", &k->cols);
}

int reduce_pass(const ReduceKernels &k, const void *in, void *out, size_t outer, size_t R, size_t inner, size_t esize,
                hipFunction_t rows_plain = nullptr)
{
    const hipFunction_t rows = k.rows, rows4 = k.rows4, cols = k.cols;
    if (!rows_plain) rows_plain = rows;
    if (outer * inner == 0) return DOPT_HIP_OK;
    if (inner > 1 || R <= 64) {
        unsigned grid = grid_for(256, outer * inner);
        void *args[] = {(void *)&in, (void *)&out, (void *)&outer, (void *)&R, (void *)&inner};
        return rtc_launch(cols, grid, 256, args);
    }
    // contiguous rows
    size_t nchunks = 1;
    if (outer < 1024) {
        size_t want = ceil_div((size_t)num_cus() * 4, outer);
        size_t maxc = ceil_div(R, (size_t)256 * 16);
        nchunks = want < maxc ? want : maxc;
        if (nchunks < 1) nchunks = 1;
    }
    size_t chunk = ceil_div(R, nchunks);
    chunk = (chunk + 1023) / 1024 * 1024;
    nchunks = ceil_div(R, chunk);
    hipFunction_t first = R % 4 == 0 ? (aligned16(in) ? rows4 : k.rows4u) : rows;
    if (nchunks == 1) {
        void *args[] = {(void *)&in, (void *)&out, (void *)&R, (void *)&chunk, (void *)&nchunks};
        return rtc_launch(first, (unsigned)outer, 256, args);
    }
    // the partial results live in the process-wide scratch (one in-order stream: no reuse hazard)
    void *partial = workspace(outer * nchunks * esize);
    if (!partial) return DOPT_HIP_ERR_OOM;
    {
        void *args[] = {(void *)&in, (void *)&partial, (void *)&R, (void *)&chunk, (void *)&nchunks};
        if (int rc = rtc_launch(first, (unsigned)(outer * nchunks), 256, args)) return rc;
    }
    size_t one = 1, r2 = nchunks, chunk2 = (nchunks + 255) / 256 * 256;
    const void *pin = partial;
    void *args[] = {(void *)&pin, (void *)&out, (void *)&r2, (void *)&chunk2, (void *)&one};
    return rtc_launch(rows_plain, (unsigned)outer, 256, args);
}

}  // namespace

extern "C" {

int dopt_hip_pointwise(const char *op, int dtype, size_t n, const void *a, const void *b, void *out)
{
    DOPT_REQUIRE(op != nullptr, "dopt_hip_pointwise: op is null");
    const OpInfo *info = find_op(op);
    if (!info) return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_pointwise: unknown operation '%s'", op);
    if (int rc = check_dtype(dtype)) return rc;
    if (n == 0) return DOPT_HIP_OK;   // empty tensors have no buffers: nothing to check them against
    DOPT_REQUIRE((info->arity == 2) == (b != nullptr), "dopt_hip_pointwise: '%s' takes %d operand(s)", op,
                 info->arity);
    DOPT_REQUIRE(a && out, "dopt_hip_pointwise: null operand");
    DOPT_ENSURE_INIT();
    bool vec = aligned16(a) && aligned16(out) && (!b || aligned16(b));
    const char *kname = vec ? "pw_vec" : "pw_scalar";
    std::string key = std::string("pw:") + op + (dtype == DOPT_HIP_F32 ? ":f32:" : ":i32:") + kname;
    hipFunction_t fn;
    if (int rc = rtc_get(key, pointwise_source(*info, dtype), kname, &fn)) return rc;
    const void *bb = b ? b : a;
    unsigned grid = vec ? grid_for(256 * 4, ceil_div(n, 4)) : grid_for(256, n);
    void *args[] = {(void *)&n, (void *)&a, (void *)&bb, (void *)&out};
    return rtc_launch(fn, grid, 256, args);
}

// Checks a chain description and produces its cache key and source.
static int chain_prepare(int dtype, int nin, const unsigned char *in_is_scalar, int nnodes, const char *const *node_op,
                         const int *node_lhs, const int *node_rhs, std::string *key, std::string *source)
{
    DOPT_REQUIRE(nin >= 1 && nin <= 16 && nnodes >= 1 && nnodes <= 64, "dopt_hip_pointwise_chain: %d inputs, %d nodes", nin,
                 nnodes);
    DOPT_REQUIRE(in_is_scalar && node_op && node_lhs && node_rhs, "dopt_hip_pointwise_chain: null argument");
    if (int rc = check_dtype(dtype)) return rc;
    const OpInfo *ops[64];
    *key = dtype == DOPT_HIP_F32 ? "chain:f32" : "chain:i32";
    for (int k = 0; k < nin; k++) {
        DOPT_REQUIRE(in_is_scalar[k] <= 3, "dopt_hip_pointwise_chain: input %d has unknown kind %d", k, (int)in_is_scalar[k]);
        *key += in_is_scalar[k] == 0 ? ":v" : in_is_scalar[k] == 1 ? ":s" : in_is_scalar[k] == 2 ? ":r" : ":c";
    }
    for (int j = 0; j < nnodes; j++) {
        DOPT_REQUIRE(node_op[j] != nullptr, "dopt_hip_pointwise_chain: node %d has no operation", j);
        ops[j] = find_op(node_op[j]);
        if (!ops[j]) return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_pointwise_chain: unknown operation '%s'", node_op[j]);
        const int limit = nin + j;   // a node may only read inputs and earlier nodes
        DOPT_REQUIRE(node_lhs[j] >= 0 && node_lhs[j] < limit && (ops[j]->arity == 1 || (node_rhs[j] >= 0 && node_rhs[j] < limit)),
                     "dopt_hip_pointwise_chain: node %d reads an operand that is not computed before it", j);
        *key += std::string("|") + node_op[j] + "," + std::to_string(node_lhs[j]) + "," +
                std::to_string(ops[j]->arity == 2 ? node_rhs[j] : -1);
    }
    *source = chain_source(dtype, nin, in_is_scalar, nnodes, ops, node_lhs, node_rhs);
    return DOPT_HIP_OK;
}

int dopt_hip_pointwise_chain(int dtype, size_t n, size_t inner, int nin, const void *const *in,
                             const unsigned char *in_is_scalar, int nnodes, const char *const *node_op, const int *node_lhs,
                             const int *node_rhs, void *out)
{
    std::string key, source;
    if (int rc = chain_prepare(dtype, nin, in_is_scalar, nnodes, node_op, node_lhs, node_rhs, &key, &source)) return rc;
    if (n == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(in && out, "dopt_hip_pointwise_chain: null argument");
    bool vec = aligned16(out), grid_kinds = false;
    for (int k = 0; k < nin; k++) {
        DOPT_REQUIRE(in[k] != nullptr, "dopt_hip_pointwise_chain: input %d is null", k);
        grid_kinds = grid_kinds || in_is_scalar[k] >= 2;
        vec = vec && (in_is_scalar[k] == 1 || in_is_scalar[k] == 2 || aligned16(in[k]));
    }
    if (grid_kinds) {
        DOPT_REQUIRE(inner > 0 && n % inner == 0, "dopt_hip_pointwise_chain: %zu elements are not rows of %zu", n, inner);
        vec = vec && inner % 4 == 0;
    } else {
        inner = n;
    }
    DOPT_ENSURE_INIT();
    const char *kname = vec ? "chain_vec" : "chain_scalar";
    hipFunction_t fn;
    if (int rc = rtc_get(key + ":" + kname, source, kname, &fn)) return rc;
    const void *ptrs[16];
    void *args[19];
    args[0] = (void *)&n;
    args[1] = (void *)&inner;
    for (int k = 0; k < nin; k++) {
        ptrs[k] = in[k];
        args[2 + k] = (void *)&ptrs[k];
    }
    args[2 + nin] = (void *)&out;
    unsigned grid = vec ? grid_for(256, ceil_div(n, 4)) : grid_for(256, n);
    return rtc_launch(fn, grid, 256, args);
}

int dopt_hip_pointwise_chain_compile_only(int dtype, int nin, const unsigned char *in_is_scalar, int nnodes,
                                          const char *const *node_op, const int *node_lhs, const int *node_rhs,
                                          const char *arch)
{
    DOPT_REQUIRE(arch != nullptr, "dopt_hip_pointwise_chain_compile_only: null argument");
    std::string key, source;
    if (int rc = chain_prepare(dtype, nin, in_is_scalar, nnodes, node_op, node_lhs, node_rhs, &key, &source)) return rc;
    return rtc_compile_only(source, arch, nullptr);
}

int dopt_hip_pointwise_index(const char *op)
{
    if (!op) return -1;
    int i = 0;
    for (const OpInfo &o : kOps) {
        if (!strcmp(o.name, op)) return i;
        i++;
    }
    return -1;
}

int dopt_hip_pointwise_arity(const char *op)
{
    const OpInfo *info = op ? find_op(op) : nullptr;
    return info ? info->arity : 0;
}

}  // extern "C"

namespace {

// `square`: what is folded is each element's square, rounded to fp32 before it is added (sum only).
int reduce_impl(const char *op, int dtype, const size_t *shape, int rank, const size_t *axes, int naxes, const void *in,
                void *out, bool square)
{
    DOPT_REQUIRE(op && shape && axes, "dopt_hip_reduce: null argument");
    bool is_sum = !strcmp(op, "sum");
    if (!is_sum && strcmp(op, "maxElement"))
        return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_reduce: unknown reduction '%s'", op);
    if (int rc = check_dtype(dtype)) return rc;
    DOPT_REQUIRE(rank >= 1 && rank <= 16 && naxes >= 1 && naxes <= rank, "dopt_hip_reduce: bad rank/axes count");
    bool reduced[16] = {false};
    for (int i = 0; i < naxes; i++) {
        DOPT_REQUIRE(axes[i] < (size_t)rank && !reduced[axes[i]], "dopt_hip_reduce: axes must be distinct and < rank");
        reduced[axes[i]] = true;
    }
    size_t cur[16];
    size_t vol = 1;
    for (int i = 0; i < rank; i++) {
        cur[i] = shape[i];
        vol *= shape[i];
    }
    if (vol == 0) {
        // Nothing to fold.  Where only reduced axes are empty the result still has elements: the fold's start value
        // (cpu/math.d:90-247 starts a sum at 0 and a maximum at -T.max).
        size_t kept = 1;
        for (int i = 0; i < rank; i++)
            if (!reduced[i]) kept *= shape[i];
        if (kept == 0) return DOPT_HIP_OK;
        DOPT_REQUIRE(out != nullptr, "dopt_hip_reduce: null argument");
        if (is_sum) return dopt_hip_memset(out, 0, kept * 4);   // also the sum of no squares
        std::vector<uint32_t> start(kept);
        const float lowest = -std::numeric_limits<float>::max();
        uint32_t bits;
        std::memcpy(&bits, &lowest, 4);
        for (uint32_t &v : start) v = dtype == DOPT_HIP_F32 ? bits : (uint32_t)(-std::numeric_limits<int32_t>::max());
        return dopt_hip_copy_h2d(out, start.data(), kept * 4);
    }
    DOPT_REQUIRE(in && out, "dopt_hip_reduce: null argument");
    DOPT_ENSURE_INIT();

    // Runs of adjacent reduced axes collapse into one (outer, R, inner) pass each, last run first.
    // The result is independent of the order in which axes are folded up to fp32 rounding.
    std::vector<std::pair<int, int>> runs;
    for (int i = 0; i < rank;) {
        if (!reduced[i]) { i++; continue; }
        int j = i;
        while (j + 1 < rank && reduced[j + 1]) j++;
        runs.push_back({i, j});
        i = j + 1;
    }
    // fp32 sum over everything but one run of axes in the middle ([N, C, inner] -> [C], the shape of a
    // per-channel statistic): one launch instead of one pass per run of reduced axes
    if (is_sum && !square && dtype == DOPT_HIP_F32 && runs.size() == 2 && runs[0].first == 0 && runs[1].second == rank - 1) {
        size_t N = 1, C = 1, inner = 1;
        for (int i = 0; i <= runs[0].second; i++) N *= cur[i];
        for (int i = runs[0].second + 1; i < runs[1].first; i++) C *= cur[i];
        for (int i = runs[1].first; i < rank; i++) inner *= cur[i];
        int crc = DOPT_HIP_OK;
        if (channel_sum(N, C, inner, (const float *)in, (float *)out, &crc)) return crc;
    }
    std::string key = std::string("red:") + op + (dtype == DOPT_HIP_F32 ? ":f32" : ":i32");
    std::string src = reduce_source(is_sum, dtype);
    ReduceKernels plain{}, squares{};   // `squares`: the first pass of a sum of squares
    if (int rc = reduce_kernels(key, src, &plain)) return rc;
    if (square)
        if (int rc = reduce_kernels("red:sumsq:f32", reduce_source(true, dtype, true), &squares)) return rc;
    const void *src_ptr = in;
    void *tmp_prev = nullptr;
    int rc = DOPT_HIP_OK;
    for (int ri = (int)runs.size() - 1; ri >= 0 && !rc; ri--) {
        int a0 = runs[ri].first, a1 = runs[ri].second;
        size_t outer = 1, R = 1, inner = 1;
        for (int i = 0; i < a0; i++) outer *= cur[i];
        for (int i = a0; i <= a1; i++) R *= cur[i];
        for (int i = a1 + 1; i < rank; i++) inner *= cur[i];
        void *dst = out;
        void *tmp = nullptr;
        if (ri > 0) {
            rc = scratch_alloc(&tmp, outer * inner * 4);   // every element is written by the pass below: no fill
            if (rc) break;
            dst = tmp;
        }
        const bool first = square && ri == (int)runs.size() - 1;   // only what is read from `in` is squared
        rc = first ? reduce_pass(squares, src_ptr, dst, outer, R, inner, 4, plain.rows)
                   : reduce_pass(plain, src_ptr, dst, outer, R, inner, 4);
        if (tmp_prev) dopt_hip_free(tmp_prev);
        tmp_prev = tmp;
        src_ptr = dst;
        for (int i = a0; i <= a1; i++) cur[i] = 1;
    }
    if (tmp_prev) dopt_hip_free(tmp_prev);
    return rc;
}

}  // namespace

extern "C" {

int dopt_hip_reduce(const char *op, int dtype, const size_t *shape, int rank, const size_t *axes, int naxes,
                    const void *in, void *out)
{
    return reduce_impl(op, dtype, shape, rank, axes, naxes, in, out, false);
}

int dopt_hip_reduce_squares(const size_t *shape, int rank, const size_t *axes, int naxes, const float *in, float *out)
{
    DOPT_REQUIRE(shape && axes, "dopt_hip_reduce_squares: null argument");
    DOPT_REQUIRE(rank >= 1 && rank <= 16 && naxes >= 1 && naxes <= rank, "dopt_hip_reduce_squares: bad rank/axes count");
    // One run of adjacent reduced axes is one pass that squares on load.  Several runs take dopt_hip_reduce's own route
    // (which has a kernel of its own for sums around a kept run of axes), on the stored product: same value either way.
    bool reduced[16] = {false};
    for (int i = 0; i < naxes; i++)
        if (axes[i] < (size_t)rank) reduced[axes[i]] = true;
    int runs = 0;
    size_t vol = 1;
    for (int i = 0; i < rank; i++) {
        vol *= shape[i];
        if (reduced[i] && (i == 0 || !reduced[i - 1])) runs++;
    }
    if (runs <= 1 || vol == 0) return reduce_impl("sum", DOPT_HIP_F32, shape, rank, axes, naxes, in, out, true);
    DOPT_REQUIRE(in && out, "dopt_hip_reduce_squares: null argument");
    void *product = nullptr;
    if (int rc = scratch_alloc(&product, vol * sizeof(float))) return rc;
    int rc = dopt_hip_pointwise("mul", DOPT_HIP_F32, vol, in, in, product);
    if (!rc) rc = reduce_impl("sum", DOPT_HIP_F32, shape, rank, axes, naxes, product, out, false);
    dopt_hip_free(product);
    return rc;
}

int dopt_hip_argmin(int dtype, const size_t *shape, int rank, size_t axis, const void *in, int32_t *out)
{
    DOPT_REQUIRE(shape && in && out, "dopt_hip_argmin: null argument");
    if (int rc = check_dtype(dtype)) return rc;
    DOPT_REQUIRE(rank >= 1 && rank <= 16 && axis < (size_t)rank, "dopt_hip_argmin: axis must be < rank");
    size_t outer = 1, A = shape[axis], vol = 1;
    for (size_t i = 0; i < axis; i++) outer *= shape[i];
    for (int i = (int)axis + 1; i < rank; i++) vol *= shape[i];
    if (outer * vol == 0) return DOPT_HIP_OK;
    DOPT_ENSURE_INIT();
    hipFunction_t fn;
    std::string key = std::string("argmin") + (dtype == DOPT_HIP_F32 ? ":f32" : ":i32");
    if (vol == 1 && A >= 64 && A < 0x7fffffffu) {
        const bool vec = A % 4 == 0 && A >= 256 && aligned16(in);
        if (int rc = rtc_get(key + (vec ? ":rows4" : ":rows"), argmin_source(dtype), vec ? "argmin_rows4_k" : "argmin_rows_k", &fn))
            return rc;
        void *rargs[] = {(void *)&in, (void *)&out, (void *)&outer, (void *)&A};
        return rtc_launch(fn, (unsigned)ceil_div(outer, (size_t)4), 256, rargs);
    }
    if (int rc = rtc_get(key, argmin_source(dtype), "argmin_k", &fn)) return rc;
    unsigned grid = grid_for(256, outer * vol);
    void *args[] = {(void *)&in, (void *)&out, (void *)&outer, (void *)&A, (void *)&vol};
    return rtc_launch(fn, grid, 256, args);
}

int dopt_hip_rtc_compile_only(const char *op, int dtype, const char *arch)
{
    DOPT_REQUIRE(op && arch, "dopt_hip_rtc_compile_only: null argument");
    if (int rc = check_dtype(dtype)) return rc;
    std::string src;
    if (!strcmp(op, "sum") || !strcmp(op, "maxElement")) {
        src = reduce_source(!strcmp(op, "sum"), dtype);
    } else if (!strcmp(op, "sumOfSquares")) {   // the first pass of dopt_hip_reduce_squares
        src = reduce_source(true, DOPT_HIP_F32, true);
    } else if (!strcmp(op, "argmin")) {
        src = argmin_source(dtype);
    } else {
        const OpInfo *info = find_op(op);
        if (!info) return fail(DOPT_HIP_ERR_UNSUPPORTED, "dopt_hip_rtc_compile_only: unknown operation '%s'", op);
        src = pointwise_source(*info, dtype);
    }
    return rtc_compile_only(src, arch, nullptr);
}

}  // extern "C"
