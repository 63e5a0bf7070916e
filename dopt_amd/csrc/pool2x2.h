// The 2 x 2 max-pool rules shared by the stand-alone kernels (nn.hip) and the batch-norm kernels
// that carry a pooling step (bn.hip).  std.algorithm.max(acc, v) = acc < v ? v : acc, starting from
// -float.max, over the window in row-major order (cpu/source/dopt/cpu/nnet.d:103-113).
#pragma once
#include <cfloat>
#include <hip/hip_runtime.h>

namespace dopt {

__device__ inline float dmax(float acc, float v) { return acc < v ? v : acc; }

// The value of a window (a b / c d).
__device__ inline float pool2x2(float a, float b, float c, float d)
{
    return dmax(dmax(dmax(dmax(-FLT_MAX, a), b), c), d);
}

// Gradient goes to the element the forward pass selected: the same chain of `acc < v` tests starting from
// -FLT_MAX, in row-major order, so the first maximum wins and an element that never compares greater (a NaN)
// is never selected; a window in which nothing fires sends its gradient to its first element.
__device__ inline void route2x2(float a, float b, float c, float d, float g, float &oa, float &ob, float &oc,
                                float &od)
{
    int best = 0;
    float bv = -FLT_MAX;
    if (bv < a) { bv = a; best = 0; }
    if (bv < b) { bv = b; best = 1; }
    if (bv < c) { bv = c; best = 2; }
    if (bv < d) { bv = d; best = 3; }
    oa = best == 0 ? g : 0.0f;
    ob = best == 1 ? g : 0.0f;
    oc = best == 2 ? g : 0.0f;
    od = best == 3 ? g : 0.0f;
}

}  // namespace dopt
