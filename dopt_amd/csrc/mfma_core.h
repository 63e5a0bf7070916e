// fp32 MFMA tile engine shared by the SGEMM and the implicit-GEMM convolution kernels.
//
// A workgroup of WM x WN wavefronts owns a BM x BN output tile; each wavefront owns a
// (BM/WM) x (BN/WN) sub-tile held as MI x NI accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs
// each).  Operand slabs of BK reduction steps are staged in LDS k-major -- As[k][m], Bs[k][n] --
// so that the fragment a lane feeds to the matrix core (A: row = lane % 32, k = lane / 32; B:
// col = lane % 32, k = lane / 32) is one conflict-free ds_read_b32.  LDS is double buffered: the
// next slab is fetched from global memory into registers while the current one is multiplied,
// then written to the other buffer, so each slab costs one barrier.
#pragma once

#include <hip/hip_runtime.h>

namespace dopt {

typedef float v16f __attribute__((ext_vector_type(16)));

template <int BM_, int BN_, int WM_, int WN_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    static constexpr int THREADS = 64 * WM * WN;
    static constexpr int MI = BM / WM / 32, NI = BN / WN / 32;  // 32x32 accumulators per wavefront
    static constexpr int LDA = BM + 4, LDB = BN + 4;             // LDS row strides (floats), 16-byte aligned rows
};

// Multiplies one LDS slab into the wavefront's accumulators.
//   As, Bs : slab bases;  a_off/b_off : the wavefront's first row / column inside the block tile.
// Software pipelined: the fragments of step ks+1 are requested from LDS before the MFMAs of step
// ks are issued, so the LDS latency hides behind the matrix work.
template <int BK, int LDA, int LDB, int MI, int NI>
__device__ inline void mma_slab(const float *As, const float *Bs, int a_off, int b_off, v16f (&acc)[MI][NI], int lane)
{
    const int kh = lane >> 5, l32 = lane & 31;
    const float *ap = As + kh * LDA + a_off + l32;
    const float *bp = Bs + kh * LDB + b_off + l32;
    float a[MI], b[NI];
#pragma unroll
    for (int i = 0; i < MI; i++) a[i] = ap[32 * i];
#pragma unroll
    for (int j = 0; j < NI; j++) b[j] = bp[32 * j];
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
        float na[MI], nb[NI];
#pragma unroll
        for (int i = 0; i < MI; i++) na[i] = ks + 1 < BK / 2 ? ap[(2 * ks + 2) * LDA + 32 * i] : 0.0f;
#pragma unroll
        for (int j = 0; j < NI; j++) nb[j] = ks + 1 < BK / 2 ? bp[(2 * ks + 2) * LDB + 32 * j] : 0.0f;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < MI; i++) a[i] = na[i];
#pragma unroll
        for (int j = 0; j < NI; j++) b[j] = nb[j];
    }
}


// Compile-time loop: f(StepTag<I>{}) for I = 0 .. N-1, so that the body can use I in constant
// expressions (register-array indices, `if constexpr`).
template <int I>
struct StepTag {
    static constexpr int value = I;
};

template <int I, int N, class F>
__device__ inline void static_for(F &&f)
{
    if constexpr (I < N) {
        f(StepTag<I>{});
        static_for<I + 1, N>(f);
    }
}

template <int MI, int NI>
__device__ inline void zero_acc(v16f (&acc)[MI][NI])
{
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
}

// Row of accumulator register v of a 32x32 tile for this lane; the column is lane % 32.
__device__ inline int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

// Workgroup ids are handed to the 8 XCDs round-robin and each XCD has its own L2.  Remap so that
// every XCD works on one contiguous range of logical ids: work items that share an operand
// (adjacent logical ids) then hit the same L2.  Returns false for the padding ids past `total`.
__device__ inline bool xcd_remap(unsigned bid, unsigned total, unsigned *logical)
{
    const unsigned per = (total + 7u) / 8u;
    const unsigned l = (bid & 7u) * per + (bid >> 3);
    *logical = l;
    return l < total;
}

inline unsigned xcd_grid(unsigned total) { return ((total + 7u) / 8u) * 8u; }

// Buffer-resource loads: the hardware range check returns 0 for an offset at or past the end of
// the buffer, so a masked element is loaded from kOobOffset instead of being branched around.
// That keeps the gather loops branch-free (one basic block the scheduler can interleave with the
// MFMAs) and the address arithmetic 32-bit.  Valid byte offsets must stay below 2^31, and a masked
// lane must carry exactly kOobOffset: the wave-uniform offset is added to it without wrapping.
constexpr unsigned kOobOffset = 0x80000000u;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void *base, size_t bytes)
{
    const size_t clamped = bytes < 0x7fffffffu ? bytes : 0x7fffffffu;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)clamped, 0x00020000);
}

// voffset: per-lane byte offset (VGPR); soffset: wave-uniform byte offset (SGPR).
__device__ inline float buffer_load_f32(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voffset, (int)soffset, 0));
}

__device__ inline float4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset)
{
    // Keep the builtin's own vector type: converting it to an ext_vector_type first makes the
    // compiler load a single dword and splat it.
    auto v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voffset, (int)soffset, 0);
    static_assert(sizeof(v) == sizeof(float4), "b128 load must yield 16 bytes");
    return __builtin_bit_cast(float4, v);
}

}  // namespace dopt
