// fp32 MFMA tile engine shared by the SGEMM and the implicit-GEMM convolution kernels.
//
// A workgroup of 256 threads (4 wavefronts of 64) owns a BM x BN output tile; each wavefront
// owns a 64 x 64 sub-tile held as 2 x 2 accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs each).
// Operand slabs of BK reduction steps are staged in LDS k-major -- As[k][m], Bs[k][n] -- so that
// the fragment a lane feeds to the matrix core (A: row = lane % 32, k = lane / 32; B: col =
// lane % 32, k = lane / 32) is one conflict-free ds_read_b32.  LDS is double buffered: the next
// slab is fetched from global memory into registers while the current one is multiplied, then
// written to the other buffer, so each slab costs one barrier.
#pragma once

#include <hip/hip_runtime.h>

namespace dopt {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;

// Multiplies one LDS slab into the wavefront's accumulators.
//   As, Bs : slab bases;  lda/ldb : row strides in floats;  a_off/b_off : the wavefront's first
//   row / column inside the block tile.
template <int BK, int LDA, int LDB>
__device__ inline void mma_slab(const float *As, const float *Bs, int a_off, int b_off, v16f (&acc)[2][2], int lane)
{
    const int kh = lane >> 5, l32 = lane & 31;
    const float *ap = As + kh * LDA + a_off + l32;
    const float *bp = Bs + kh * LDB + b_off + l32;
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
        float a0 = ap[(2 * ks) * LDA], a1 = ap[(2 * ks) * LDA + 32];
        float b0 = bp[(2 * ks) * LDB], b1 = bp[(2 * ks) * LDB + 32];
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
}

__device__ inline void zero_acc(v16f (&acc)[2][2])
{
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
}

// Row of accumulator register v of a 32x32 tile for this lane; the column is lane % 32.
__device__ inline int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

// Workgroup ids are handed to the 8 XCDs round-robin and each XCD has its own L2.  Remap so that
// every XCD works on one contiguous range of logical tiles: tiles that share an operand (adjacent
// logical ids) then hit the same L2.  Returns false for the padding ids past `total`.
__device__ inline bool xcd_remap(unsigned bid, unsigned total, unsigned *logical)
{
    const unsigned per = (total + 7u) / 8u;
    const unsigned l = (bid & 7u) * per + (bid >> 3);
    *logical = l;
    return (bid >> 3) < per && l < total;
}

inline unsigned xcd_grid(unsigned total) { return ((total + 7u) / 8u) * 8u; }

}  // namespace dopt
