// A run of operations on tiny tensors as ONE launch of ONE workgroup.
//
// The tail of a training graph - softmax, the loss's logarithm, product with the labels, sum, scaling, and the way
// back through the same operations - is a chain of kernels on a few hundred values each.  Every one of them lasts as
// long as a kernel boundary does (4-5 us between dependent kernels of one queue), whatever it computes.  Here a
// single block of 256 threads walks the chain: node after node, each node's elements dealt over the threads, a
// workgroup barrier between nodes, every value in the buffer the plan gave its operation (so anything outside the run
// that reads one finds it where it always was).
//
// Each node computes exactly what its stand-alone kernel computes, in the same order:
//   pointwise     the expression of pw_ops.h, one rounding (the stand-alone kernels are compiled from the same text);
//   sum/maxElement over one run of adjacent axes, as dopt_hip_reduce folds a small tensor: a strided or short
//                 reduction by one thread per output element in ascending order (red_cols), a contiguous row of more
//                 than 64 values by the whole block in the order of red_rows / red_rows4 (four chains per thread,
//                 wavefront shuffles, wavefronts in order);
//   softmax(Grad) one thread per (n, inner) lane, channels in the order of cpu/nnet.d:129-166 (softmax_fwd_k,
//                 softmax_bwd_k of nn.hip, which rows of fewer than 64 classes take);
//   repeat        a copy (core/ops/basic.d:336-356).
// So a plan that runs such a chain as one launch returns the bits of the plan that runs it kernel by kernel.
#include <vector>

#include "common.h"
#include "pool2x2.h"
#include "pw_ops.h"

namespace {

using namespace dopt;

constexpr int kTinyBlock = 256;      // threads that fold a row, as the stand-alone reduction's block does
constexpr int kTinyThreads = 1024;   // threads of the workgroup: a thread's elements run one after the other, so more threads, less time

// Pointers into device memory say so in their type: a pointer of unknown kind makes the compiler use instructions that
// serve both memory and LDS, and an LDS read then waits for every store to memory issued before it.
typedef __attribute__((address_space(1))) float gfloat;

enum PwOp {
#define DOPT_PW_ENUM(name, arity, f32, i32) OP_##name,
    DOPT_PW_OPS(DOPT_PW_ENUM)
#undef DOPT_PW_ENUM
    OP_count
};

// One loop per operation and per way of finding the operands: a thread runs a node's elements one after the other, so
// what counts is the number of instructions per element - a switch over the operation or a division for the operand
// index inside the loop costs more than the operation itself.
template <int kOp>
__device__ __forceinline__ float pw_apply(float a, float b)
{
    typedef float T;
    (void)b;
#define DOPT_PW_CASE(name, arity, f32, i32) \
    if constexpr (kOp == OP_##name) return (T)(f32);
    DOPT_PW_OPS(DOPT_PW_CASE)
#undef DOPT_PW_CASE
    return a;
}

template <int kOp, class AP>
__device__ __forceinline__ void pw_loop(int n, AP a, AP b, int ka, int kb, int inner, float *dstL, gfloat *dstG)
{
    if (ka < 2 && kb < 2) {   // element i or the only element: a stride of 1 or 0
        const int sa = ka == 0, sb = kb == 0;
        for (int i = threadIdx.x; i < n; i += kTinyThreads) {
            const float r = pw_apply<kOp>(a[i * sa], b[i * sb]);
            if (dstL) dstL[i] = r;
            if (dstG) dstG[i] = r;
        }
        return;
    }
    for (int i = threadIdx.x; i < n; i += kTinyThreads) {   // 2 at its row, 3 at its column of [n / inner, inner]
        const int row = i / inner, col = i - row * inner;
        const float r = pw_apply<kOp>(a[ka == 0 ? i : ka == 1 ? 0 : ka == 2 ? row : col], b[kb == 0 ? i : kb == 1 ? 0 : kb == 2 ? row : col]);
        if (dstL) dstL[i] = r;
        if (dstG) dstG[i] = r;
    }
}

// Everything a node reads comes from LDS.  A load from memory waits for every store the wavefront issued before it
// (one counter tracks both), so a node that reads what the node before it has just stored to memory waits for that
// store to reach the L2 and for its own load to come back: 3-4 us per node, and a chain of thirteen nodes took as long
// as the thirteen kernels it replaced.  So the host gives every operand a place in a 48 KB arena: values that enter the
// run from outside are copied in once, before the first node; a result is written to its place for as long as a node
// of the run still reads it, and to its buffer in memory as well (for whoever reads it after the run) without anyone
// waiting for that store.  A run whose operands do not all find room (first fit, places given back after their last
// reader) runs through memory instead: same values, slower.
constexpr int kArenaFloats = 12288;
constexpr int kTinyStaged = 16;
struct TinyLds {
    short dst, a, b;   // float offsets into the arena, or -1
    short pad;
};
struct TinyStage {
    const float *src;
    short at;          // float offset into the arena
    short n;
    int pad;
};
struct TinyProgram {
    void *slot[DOPT_HIP_TINY_SLOTS];
    dopt_hip_tiny_node node[DOPT_HIP_TINY_NODES];
    TinyLds lds[DOPT_HIP_TINY_NODES];
    int nnodes;
};
struct TinyStaging {
    TinyStage in[kTinyStaged];
    int n;
};

template <bool kSum>
__device__ inline float fold(float a, float b)
{
    if (kSum) return a + b;
    return (a < b || a != a) ? b : a;   // a maximum that passes over NaNs, as the stand-alone kernel's
}

template <bool kSum>
__device__ inline float fold4(float4 v)
{
    return fold<kSum>(fold<kSum>(v.x, v.y), fold<kSum>(v.z, v.w));
}

// One contiguous row of R > 64 values folded by the block exactly as block `o` of red_rows / red_rows4 folds it
// (one chunk: rows of at most 4096 values are never cut).  Every thread must call it.
template <bool kSum, class AP>
__device__ __forceinline__ void reduce_row(AP row, int R, bool quads, float *out, gfloat *out2, float *part)
{
    const float ident = kSum ? 0.0f : -3.402823466e+38f;
    float acc0 = ident, acc1 = ident, acc2 = ident, acc3 = ident;
    const int B = kTinyBlock;
    const bool on = threadIdx.x < B;   // the first 256 threads are the stand-alone kernel's block; the others keep the barriers company
    if (!on) {
    } else if (quads) {
        auto quad = [&](int q) { return make_float4(row[4 * q], row[4 * q + 1], row[4 * q + 2], row[4 * q + 3]); };
        const int q1 = R / 4;
        int i = threadIdx.x;
        for (; i + 3 * B < q1; i += 4 * B) {
            const float4 v0 = quad(i), v1 = quad(i + B), v2 = quad(i + 2 * B), v3 = quad(i + 3 * B);
            acc0 = fold<kSum>(acc0, fold4<kSum>(v0));
            acc1 = fold<kSum>(acc1, fold4<kSum>(v1));
            acc2 = fold<kSum>(acc2, fold4<kSum>(v2));
            acc3 = fold<kSum>(acc3, fold4<kSum>(v3));
        }
        for (; i < q1; i += B) acc0 = fold<kSum>(acc0, fold4<kSum>(quad(i)));
    } else {
        int i = threadIdx.x;
        for (; i + 3 * B < R; i += 4 * B) {
            const float v0 = row[i], v1 = row[i + B], v2 = row[i + 2 * B], v3 = row[i + 3 * B];
            acc0 = fold<kSum>(acc0, v0);
            acc1 = fold<kSum>(acc1, v1);
            acc2 = fold<kSum>(acc2, v2);
            acc3 = fold<kSum>(acc3, v3);
        }
        for (; i < R; i += B) acc0 = fold<kSum>(acc0, row[i]);
    }
    float v = fold<kSum>(fold<kSum>(acc0, acc1), fold<kSum>(acc2, acc3));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_down(v, off, 64);
        v = fold<kSum>(v, o);
    }
    __syncthreads();   // `part` may still be read from the row before
    if (on && (threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kTinyBlock / 64; w++) v = fold<kSum>(v, part[w]);
        if (out) *out = v;
        if (out2) *out2 = v;
    }
}

template <bool kSum, class AP>
__device__ __forceinline__ void reduce_node(const dopt_hip_tiny_node &nd, AP in, bool in_aligned, float *out, gfloat *out2, float *part)
{
    const int outer = nd.dims[0], R = nd.dims[1], inner = nd.dims[2];
    if (inner > 1 || R <= 64) {   // red_cols: thread (o, j) folds in ascending r from the identity
        const float ident = kSum ? 0.0f : -3.402823466e+38f;
        for (int idx = threadIdx.x; idx < outer * inner; idx += kTinyThreads) {
            const int o = idx / inner, j = idx - o * inner;
            AP p = in + (size_t)o * R * inner + j;
            float acc = ident;
            for (int r = 0; r < R; r++) acc = fold<kSum>(acc, p[(size_t)r * inner]);
            if (out) out[idx] = acc;
            if (out2) out2[idx] = acc;
        }
        return;
    }
    (void)in_aligned;
    const bool quads = R % 4 == 0;   // dopt_hip_reduce's test: the order does not depend on where the row starts in memory
    for (int o = 0; o < outer; o++) reduce_row<kSum, AP>(in + (size_t)o * R, R, quads, out ? out + o : nullptr, out2 ? out2 + o : nullptr, part);
}

// One node.  a, b: where its operands lie; dstL: the result's place in LDS (or null), dstG: its buffer in memory (or
// null).  The softmax keeps its exponentials where it will leave the result: in LDS when it has a place there.
template <class AP>
__device__ __forceinline__ void run_node(const dopt_hip_tiny_node &nd, AP a, AP b, bool a_aligned, float *dstL, gfloat *dstG,
                                         float *part)
{
    const int n = nd.n;
    switch (nd.kind) {
    case DOPT_HIP_TINY_POINTWISE: {
        // where result i finds an operand: 0 at i, 1 at its only element, 2 at its row, 3 at its column of [n / dims[0], dims[0]]
        const int inner = nd.dims[0] > 0 ? nd.dims[0] : 1;
        const int ka = nd.a_kind, kb = nd.b < 0 ? nd.a_kind : nd.b_kind;
        switch (nd.op) {
#define DOPT_PW_CASE(name, arity, f32, i32) \
        case OP_##name:                         \
            pw_loop<OP_##name, AP>(n, a, b, ka, kb, inner, dstL, dstG); \
            break;
            DOPT_PW_OPS(DOPT_PW_CASE)
#undef DOPT_PW_CASE
        }
        break;
    }
    case DOPT_HIP_TINY_REDUCE:
        if (nd.op == 0) reduce_node<true, AP>(nd, a, a_aligned, dstL, dstG, part);
        else reduce_node<false, AP>(nd, a, a_aligned, dstL, dstG, part);
        break;
    case DOPT_HIP_TINY_SOFTMAX: {
        const int N = nd.dims[0], C = nd.dims[1], inner = nd.dims[2];
        for (int idx = threadIdx.x; idx < N * inner; idx += kTinyThreads) {
            const int nn = idx / inner, i = idx - nn * inner;
            const size_t base = (size_t)nn * C * inner + i;
            AP px = a + base;
            float m = -FLT_MAX;
            if (C <= 16) {   // a short row: all its loads in flight together, then the same operations in the same order
                float x[16];
#pragma unroll
                for (int c = 0; c < 16; c++) x[c] = px[(size_t)min(c, C - 1) * inner];
#pragma unroll
                for (int c = 0; c < 16; c++)
                    if (c < C) m = dmax(m, x[c]);
                float s = 0.0f;
#pragma unroll
                for (int c = 0; c < 16; c++)
                    if (c < C) {
                        x[c] = expf(x[c] - m);
                        s += x[c];
                    }
#pragma unroll
                for (int c = 0; c < 16; c++)
                    if (c < C) {
                        const float r = x[c] / s;
                        if (dstL) dstL[base + (size_t)c * inner] = r;
                        if (dstG) dstG[base + (size_t)c * inner] = r;
                    }
                continue;
            }
            for (int c = 0; c < C; c++) m = dmax(m, px[(size_t)c * inner]);
            float s = 0.0f;
            if (dstL) {
                float *py = dstL + base;
                for (int c = 0; c < C; c++) {
                    const float pot = expf(px[(size_t)c * inner] - m);
                    s += pot;
                    py[(size_t)c * inner] = pot;
                }
                for (int c = 0; c < C; c++) {
                    const float r = py[(size_t)c * inner] / s;
                    py[(size_t)c * inner] = r;
                    if (dstG) dstG[base + (size_t)c * inner] = r;
                }
            } else {
                gfloat *py = dstG + base;
                for (int c = 0; c < C; c++) {
                    const float pot = expf(px[(size_t)c * inner] - m);
                    s += pot;
                    py[(size_t)c * inner] = pot;
                }
                for (int c = 0; c < C; c++) py[(size_t)c * inner] = py[(size_t)c * inner] / s;
            }
        }
        break;
    }
    case DOPT_HIP_TINY_SOFTMAX_GRAD: {   // a = dy, b = y
        const int N = nd.dims[0], C = nd.dims[1], inner = nd.dims[2];
        for (int idx = threadIdx.x; idx < N * inner; idx += kTinyThreads) {
            const int nn = idx / inner, i = idx - nn * inner;
            const size_t base = (size_t)nn * C * inner + i;
            float dot = 0.0f;
            if (C <= 16) {
                float g[16], y[16];
#pragma unroll
                for (int c = 0; c < 16; c++) {
                    g[c] = a[base + (size_t)min(c, C - 1) * inner];
                    y[c] = b[base + (size_t)min(c, C - 1) * inner];
                }
#pragma unroll
                for (int c = 0; c < 16; c++)
                    if (c < C) dot += g[c] * y[c];
#pragma unroll
                for (int c = 0; c < 16; c++)
                    if (c < C) {
                        const float r = y[c] * (g[c] - dot);
                        if (dstL) dstL[base + (size_t)c * inner] = r;
                        if (dstG) dstG[base + (size_t)c * inner] = r;
                    }
                continue;
            }
            for (int c = 0; c < C; c++) dot += a[base + (size_t)c * inner] * b[base + (size_t)c * inner];
            for (int c = 0; c < C; c++) {
                const float r = b[base + (size_t)c * inner] * (a[base + (size_t)c * inner] - dot);
                if (dstL) dstL[base + (size_t)c * inner] = r;
                if (dstG) dstG[base + (size_t)c * inner] = r;
            }
        }
        break;
    }
    case DOPT_HIP_TINY_REPEAT: {   // dims = the input's extents (leading 1s for ranks below 4), reps beside them
        if (nd.dims[0] * nd.dims[1] * nd.dims[2] * nd.dims[3] == 1) {   // one value, n times
            const float r = a[0];
            for (int i = threadIdx.x; i < n; i += kTinyThreads) {
                if (dstL) dstL[i] = r;
                if (dstG) dstG[i] = r;
            }
            break;
        }
        const int o1 = nd.dims[1] * nd.reps[1], o2 = nd.dims[2] * nd.reps[2], o3 = nd.dims[3] * nd.reps[3];
        for (int i = threadIdx.x; i < n; i += kTinyThreads) {
            const int c3 = i % o3, t3 = i / o3, c2 = t3 % o2, t2 = t3 / o2, c1 = t2 % o1, c0 = t2 / o1;
            const int src = (((c0 % nd.dims[0]) * nd.dims[1] + c1 % nd.dims[1]) * nd.dims[2] + c2 % nd.dims[2]) * nd.dims[3] +
                            c3 % nd.dims[3];
            const float r = a[src];   // moved as it is: no arithmetic touches it
            if (dstL) dstL[i] = r;
            if (dstG) dstG[i] = r;
        }
        break;
    }
    }
}

// Through memory: every node reads its operands from, and writes its result to, the buffers themselves.
// The run's description arrives as kernel arguments, which live in host-visible memory: read node by node as the loop
// reaches them, every node waited a microsecond or two for its own description.  All threads fetch it together instead,
// 16 bytes each, into LDS, and the loop reads it from there.
template <class T>
__device__ __forceinline__ void fetch_args(const T &args, T *to)
{
    static_assert(sizeof(T) % 4 == 0, "copied in words");
    const unsigned *src = (const unsigned *)&args;
    unsigned *dst = (unsigned *)to;
    for (unsigned i = threadIdx.x; i < sizeof(T) / 4; i += kTinyThreads) dst[i] = src[i];
}

__global__ __launch_bounds__(kTinyThreads) void tiny_graph_mem_k(TinyProgram args)
{
    __shared__ float part[kTinyBlock / 64];
    __shared__ TinyProgram pr;
    fetch_args(args, &pr);
    __syncthreads();
    for (int k = 0; k < pr.nnodes; k++) {
        const dopt_hip_tiny_node &nd = pr.node[k];
        gfloat *mem = (gfloat *)((uintptr_t)pr.slot[nd.dst] + (uintptr_t)nd.dst_offset);
        const gfloat *a = (const gfloat *)((uintptr_t)pr.slot[nd.a] + (uintptr_t)nd.a_offset);
        const gfloat *b = nd.b < 0 ? a : (const gfloat *)((uintptr_t)pr.slot[nd.b] + (uintptr_t)nd.b_offset);
        run_node<const gfloat *>(nd, a, b, ((uintptr_t)a & 15u) == 0, nullptr, mem, part);
        __syncthreads();   // the next node reads what this one wrote (stores of a workgroup are ordered by its barrier)
    }
}

// Through LDS: every operand has a place in the arena (see above).
__global__ __launch_bounds__(kTinyThreads) void tiny_graph_lds_k(TinyProgram args, TinyStaging staged)
{
    __shared__ float part[kTinyBlock / 64];
    __shared__ __attribute__((aligned(16))) float arena[kArenaFloats];
    __shared__ TinyProgram pr;
    __shared__ TinyStaging st;
    fetch_args(args, &pr);
    fetch_args(staged, &st);
    __syncthreads();
    if (st.n > 0) {   // what enters from outside: the loads of ALL ranges in flight together (one after the other, each range cost a
        // trip to memory), two per range and thread, then a loop for what is left of ranges beyond 2048 values
        float v[kTinyStaged][2];
#pragma unroll
        for (int e = 0; e < kTinyStaged; e++) {
            const int ee = min(e, st.n - 1), n = st.in[ee].n;
            const gfloat *src = (const gfloat *)(uintptr_t)st.in[ee].src;
#pragma unroll
            for (int u = 0; u < 2; u++) v[e][u] = src[min((int)threadIdx.x + u * kTinyThreads, n - 1)];
        }
#pragma unroll
        for (int e = 0; e < kTinyStaged; e++) {
            if (e >= st.n) break;
            float *to = arena + st.in[e].at;
#pragma unroll
            for (int u = 0; u < 2; u++)
                if ((int)threadIdx.x + u * kTinyThreads < st.in[e].n) to[threadIdx.x + u * kTinyThreads] = v[e][u];
        }
        for (int e = 0; e < st.n; e++) {
            const gfloat *src = (const gfloat *)(uintptr_t)st.in[e].src;
            float *to = arena + st.in[e].at;
            for (int i = threadIdx.x + 2 * kTinyThreads; i < st.in[e].n; i += kTinyThreads) to[i] = src[i];
        }
    }
    __syncthreads();
    for (int k = 0; k < pr.nnodes; k++) {
        const dopt_hip_tiny_node &nd = pr.node[k];
        const TinyLds &ld = pr.lds[k];
        gfloat *mem = (gfloat *)((uintptr_t)pr.slot[nd.dst] + (uintptr_t)nd.dst_offset);
        const float *a = arena + ld.a;
        const float *b = nd.b < 0 ? a : arena + ld.b;
        // (the row sums take quads where the tensor in memory would allow it)
        const bool aligned = (((uintptr_t)pr.slot[nd.a] + (uintptr_t)nd.a_offset) & 15u) == 0;
        run_node<const float *>(nd, a, b, aligned, ld.dst >= 0 ? arena + ld.dst : nullptr, mem, part);
        __syncthreads();
    }
}

// How many values a node reads from operand a (which = 0) or b (1).
int operand_extent(const dopt_hip_tiny_node &nd, int which)
{
    switch (nd.kind) {
    case DOPT_HIP_TINY_POINTWISE: {
        const int kind = which == 0 ? nd.a_kind : nd.b_kind, inner = nd.dims[0] > 0 ? nd.dims[0] : 1;
        return kind == 0 ? nd.n : kind == 1 ? 1 : kind == 2 ? nd.n / inner : inner;
    }
    case DOPT_HIP_TINY_REDUCE: return nd.dims[0] * nd.dims[1] * nd.dims[2];
    case DOPT_HIP_TINY_REPEAT: return nd.dims[0] * nd.dims[1] * nd.dims[2] * nd.dims[3];
    default: return nd.n;
    }
}

// Places in the arena: for every operand the latest earlier node whose result covers it (by address: two slots may
// name one buffer), or the range of memory it enters the run from; for every result the span of nodes that read it; then
// first fit in node order, places given back when their last reader has run.  False when something finds no room (or
// an operand overlaps an earlier result only in part): the run then goes through memory.
bool assign_lds(int nnodes, const dopt_hip_tiny_node *nodes, void *const *slots, TinyLds *lds, TinyStaging *st)
{
    int producer[DOPT_HIP_TINY_NODES][2], last_reader[DOPT_HIP_TINY_NODES];
    struct Ext { const char *lo, *hi; int at; };
    std::vector<Ext> exts;
    int ext_of[DOPT_HIP_TINY_NODES][2];
    for (int k = 0; k < nnodes; k++) {
        last_reader[k] = -1;
        lds[k] = TinyLds{-1, -1, -1, 0};
        for (int w = 0; w < 2; w++) {
            producer[k][w] = ext_of[k][w] = -1;
            const int slot = w == 0 ? nodes[k].a : nodes[k].b;
            if (slot < 0) continue;
            const char *lo = (const char *)slots[slot] + (w == 0 ? nodes[k].a_offset : nodes[k].b_offset);
            const char *hi = lo + (size_t)operand_extent(nodes[k], w) * 4;
            bool found = false;
            for (int j = k - 1; j >= 0 && !found; j--) {
                const char *plo = (const char *)slots[nodes[j].dst] + nodes[j].dst_offset, *phi = plo + (size_t)nodes[j].n * 4;
                if (hi <= plo || phi <= lo) continue;
                if (!(plo <= lo && hi <= phi)) return false;
                producer[k][w] = j;
                last_reader[j] = k;
                found = true;
            }
            if (found) continue;
            // from outside: one copy per distinct range (ranges that merely overlap are copied apart)
            for (size_t e = 0; e < exts.size(); e++)
                if (exts[e].lo == lo && exts[e].hi == hi) ext_of[k][w] = (int)e;
            if (ext_of[k][w] < 0) {
                exts.push_back({lo, hi, -1});
                ext_of[k][w] = (int)exts.size() - 1;
            }
        }
    }
    if (exts.size() > (size_t)kTinyStaged) return false;
    // what comes from outside stays for the whole run, at the bottom of the arena; 16-byte aligned copies of 16-byte
    // aligned ranges (a row sum reads quads from its copy exactly where it would from memory)
    int floor = 0;
    st->n = 0;
    for (Ext &e : exts) {
        const int n = (int)((e.hi - e.lo) / 4);
        const int skew = (int)(((uintptr_t)e.lo & 15u) / 4);   // the copy starts as far into a quad as the range does
        e.at = floor + skew;
        floor += (skew + n + 3) / 4 * 4;
        if (floor > kArenaFloats || n > 32767) return false;
        st->in[st->n++] = TinyStage{(const float *)e.lo, (short)e.at, (short)n, 0};
    }
    struct Span { int at, len, until; };
    std::vector<Span> held;
    for (int k = 0; k < nnodes; k++) {
        for (int w = 0; w < 2; w++) {
            short &place = w == 0 ? lds[k].a : lds[k].b;
            if (ext_of[k][w] >= 0) place = (short)exts[(size_t)ext_of[k][w]].at;
            const int j = producer[k][w];
            if (j < 0) continue;
            if (lds[j].dst < 0) return false;
            const char *lo = (const char *)slots[w == 0 ? nodes[k].a : nodes[k].b] + (w == 0 ? nodes[k].a_offset : nodes[k].b_offset);
            const char *plo = (const char *)slots[nodes[j].dst] + nodes[j].dst_offset;
            place = (short)(lds[j].dst + (lo - plo) / 4);
        }
        for (size_t i = 0; i < held.size();)   // (given back only after the node: a result never takes its own operand's place)
            if (held[i].until < k) held.erase(held.begin() + (long)i);
            else i++;
        const bool wanted = last_reader[k] >= 0 || nodes[k].kind == DOPT_HIP_TINY_SOFTMAX;   // (the softmax works in place)
        if (!wanted || nodes[k].n <= 0) continue;
        const int skew = (int)(((uintptr_t)((const char *)slots[nodes[k].dst] + nodes[k].dst_offset) & 15u) / 4);
        const int len = (skew + nodes[k].n + 3) / 4 * 4;
        int at = floor;
        bool moved = true;
        while (moved) {   // first fit past whatever is held
            moved = false;
            for (const Span &h : held)
                if (at < h.at + h.len && h.at < at + len) {
                    at = h.at + h.len;
                    moved = true;
                }
        }
        if (at + len > kArenaFloats) return false;
        lds[k].dst = (short)(at + skew);
        held.push_back({at, len, last_reader[k] >= 0 ? last_reader[k] : k});
    }
    return true;
}

}  // namespace

extern "C" {

int dopt_hip_tiny_graph(int nslots, void *const *slots, int nnodes, const dopt_hip_tiny_node *nodes)
{
    if (nnodes == 0) return DOPT_HIP_OK;
    DOPT_REQUIRE(slots && nodes, "dopt_hip_tiny_graph: null argument");
    DOPT_REQUIRE(nslots >= 1 && nslots <= DOPT_HIP_TINY_SLOTS && nnodes >= 1 && nnodes <= DOPT_HIP_TINY_NODES,
                 "dopt_hip_tiny_graph: %d buffers and %d nodes (at most %d and %d)", nslots, nnodes, DOPT_HIP_TINY_SLOTS,
                 DOPT_HIP_TINY_NODES);
    DOPT_ENSURE_INIT();
    TinyProgram pr{};
    for (int i = 0; i < nslots; i++) pr.slot[i] = slots[i];
    for (int k = 0; k < nnodes; k++) {
        const dopt_hip_tiny_node &nd = nodes[k];
        const bool binary = nd.kind == DOPT_HIP_TINY_SOFTMAX_GRAD || (nd.kind == DOPT_HIP_TINY_POINTWISE && nd.b >= 0);
        DOPT_REQUIRE(nd.kind >= DOPT_HIP_TINY_POINTWISE && nd.kind <= DOPT_HIP_TINY_REPEAT, "dopt_hip_tiny_graph: node %d has unknown kind %d", k, nd.kind);
        DOPT_REQUIRE(nd.dst >= 0 && nd.dst < nslots && nd.a >= 0 && nd.a < nslots && nd.b < nslots && (!binary || nd.b >= 0),
                     "dopt_hip_tiny_graph: node %d names a buffer that was not passed", k);
        DOPT_REQUIRE(slots[nd.dst] && slots[nd.a] && (nd.b < 0 || slots[nd.b]), "dopt_hip_tiny_graph: node %d: null buffer", k);
        DOPT_REQUIRE(nd.n >= 0 && nd.n <= DOPT_HIP_TINY_ELEMS, "dopt_hip_tiny_graph: node %d has %d elements (at most %d)", k, nd.n,
                     DOPT_HIP_TINY_ELEMS);
        DOPT_REQUIRE(nd.dst_offset >= 0 && nd.a_offset >= 0 && nd.b_offset >= 0 && nd.dst_offset % 4 == 0 && nd.a_offset % 4 == 0 && nd.b_offset % 4 == 0,
                     "dopt_hip_tiny_graph: node %d: byte offsets must be non-negative multiples of 4", k);
        if (nd.kind == DOPT_HIP_TINY_POINTWISE) {
            DOPT_REQUIRE(nd.op >= 0 && nd.op < OP_count, "dopt_hip_tiny_graph: node %d: unknown pointwise operation %d", k, nd.op);
            DOPT_REQUIRE(nd.a_kind >= 0 && nd.a_kind <= 3 && nd.b_kind >= 0 && nd.b_kind <= 3, "dopt_hip_tiny_graph: node %d: unknown operand kind", k);
            DOPT_REQUIRE((nd.a_kind < 2 && (nd.b < 0 || nd.b_kind < 2)) || (nd.dims[0] >= 1 && nd.n % nd.dims[0] == 0),
                         "dopt_hip_tiny_graph: node %d: %d elements are not rows of %d", k, nd.n, nd.dims[0]);
        } else if (nd.kind == DOPT_HIP_TINY_REDUCE) {
            DOPT_REQUIRE(nd.op == 0 || nd.op == 1, "dopt_hip_tiny_graph: node %d: reduction %d is neither sum (0) nor maxElement (1)", k, nd.op);
            DOPT_REQUIRE(nd.dims[0] >= 0 && nd.dims[1] >= 1 && nd.dims[2] >= 1 && (long long)nd.dims[0] * nd.dims[2] == nd.n &&
                             (long long)nd.dims[0] * nd.dims[1] * nd.dims[2] <= DOPT_HIP_TINY_ELEMS,
                         "dopt_hip_tiny_graph: node %d: a reduction of [%d, %d, %d] does not give %d values", k, nd.dims[0], nd.dims[1], nd.dims[2], nd.n);
        } else if (nd.kind == DOPT_HIP_TINY_REPEAT) {
            long long vol = 1;
            for (int d = 0; d < 4; d++) {
                DOPT_REQUIRE(nd.dims[d] >= 1 && nd.reps[d] >= 1, "dopt_hip_tiny_graph: node %d: extents and repetitions must be positive", k);
                vol *= (long long)nd.dims[d] * nd.reps[d];
            }
            DOPT_REQUIRE(vol == nd.n, "dopt_hip_tiny_graph: node %d: the repeated tensor does not have %d elements", k, nd.n);
        } else {
            DOPT_REQUIRE(nd.dims[0] >= 0 && nd.dims[1] >= 1 && nd.dims[2] >= 1 && (long long)nd.dims[0] * nd.dims[1] * nd.dims[2] == nd.n,
                         "dopt_hip_tiny_graph: node %d: softmax over [%d, %d, %d] does not have %d elements", k, nd.dims[0], nd.dims[1], nd.dims[2], nd.n);
        }
        pr.node[k] = nd;
        if (nd.kind == DOPT_HIP_TINY_POINTWISE && nd.dims[0] >= 1) {   // a grid of one column or one row needs no division
            dopt_hip_tiny_node &q = pr.node[k];
            const int inner = nd.dims[0], rows = nd.n / inner;
            auto plain = [&](int kind) { return kind == 2 ? (inner == 1 ? 0 : rows == 1 ? 1 : 2) : kind == 3 ? (inner == 1 ? 1 : rows == 1 ? 0 : 3) : kind; };
            q.a_kind = plain(nd.a_kind);
            q.b_kind = plain(nd.b_kind);
        }
    }
    pr.nnodes = nnodes;
    TinyStaging st{};
    if (assign_lds(nnodes, pr.node, slots, pr.lds, &st)) hipLaunchKernelGGL(tiny_graph_lds_k, dim3(1), dim3(kTinyThreads), 0, stream(), pr, st);
    else hipLaunchKernelGGL(tiny_graph_mem_k, dim3(1), dim3(kTinyThreads), 0, stream(), pr);
    DOPT_LAUNCH_CHECK();
    return DOPT_HIP_OK;
}

}  // extern "C"
