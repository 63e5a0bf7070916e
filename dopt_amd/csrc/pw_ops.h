// The pointwise operations, once: name, arity, fp32 expression, int32 expression of operands `a`, `b` of type T.
// rtc_ops.cpp turns the expressions into strings for its run-time compiled kernels, tiny.hip compiles the fp32 ones
// as they stand, so an operation means the same wherever it runs.  Semantics follow the CPU evaluator
// (cpu/source/dopt/cpu/math.d:312-437): integer arithmetic wraps, every integer unary op except neg goes through
// float and truncates back (cpu/math.d:418).  The last two are the activations of cuda/nnet/cudnn7.d:406-461 in the
// form nn.hip computes them (NaN passes through relu; reluGrad takes (dy, x)): nodes of pointwise chains.
// An expression that holds a comma is wrapped in parentheses so that it stays one macro argument.
#pragma once

#define DOPT_PW_OPS(X)                                                                                    \
    X(add, 2, a + b, (int)((unsigned)a + (unsigned)b))                                                    \
    X(sub, 2, a - b, (int)((unsigned)a - (unsigned)b))                                                    \
    X(mul, 2, a * b, (int)((unsigned)a * (unsigned)b))                                                    \
    X(div, 2, a / b, a / b)                                                                               \
    X(lt, 2, (T)(a < b), (T)(a < b))                                                                      \
    X(lte, 2, (T)(a <= b), (T)(a <= b))                                                                   \
    X(gt, 2, (T)(a > b), (T)(a > b))                                                                      \
    X(gte, 2, (T)(a >= b), (T)(a >= b))                                                                   \
    X(eq, 2, (T)(a == b), (T)(a == b))                                                                    \
    X(neq, 2, (T)(a != b), (T)(a != b))                                                                   \
    X(max, 2, (a < b ? b : a), (a < b ? b : a))                                                           \
    X(min, 2, (a < b ? a : b), (a < b ? a : b))                                                           \
    X(pow, 2, (powf(a, b)), (dopt_ipow(a, b)))                                                            \
    X(atan2, 2, (atan2f(a, b)), ((int)atan2f((float)a, (float)b)))                                        \
    X(neg, 1, -a, (int)(0u - (unsigned)a))                                                                \
    X(abs, 1, fabsf(a), (int)fabsf((float)a))                                                             \
    X(sgn, 1, (T)((a > 0) - (a < 0)), (int)(float)(((float)a > 0) - ((float)a < 0)))                      \
    X(exp, 1, expf(a), (int)expf((float)a))                                                               \
    X(log, 1, logf(a), (int)logf((float)a))                                                               \
    X(sqrt, 1, sqrtf(a), (int)sqrtf((float)a))                                                            \
    X(sin, 1, sinf(a), (int)sinf((float)a))                                                               \
    X(cos, 1, cosf(a), (int)cosf((float)a))                                                               \
    X(tan, 1, tanf(a), (int)tanf((float)a))                                                               \
    X(asin, 1, asinf(a), (int)asinf((float)a))                                                            \
    X(acos, 1, acosf(a), (int)acosf((float)a))                                                            \
    X(atan, 1, atanf(a), (int)atanf((float)a))                                                            \
    X(sinh, 1, sinhf(a), (int)sinhf((float)a))                                                            \
    X(cosh, 1, coshf(a), (int)coshf((float)a))                                                            \
    X(tanh, 1, tanhf(a), (int)tanhf((float)a))                                                            \
    X(asinh, 1, asinhf(a), (int)asinhf((float)a))                                                         \
    X(acosh, 1, acoshf(a), (int)acoshf((float)a))                                                         \
    X(atanh, 1, atanhf(a), (int)atanhf((float)a))                                                         \
    X(relu, 1, (a < 0 ? 0 : a), (a < 0 ? 0 : a))                                                          \
    X(reluGrad, 2, (b > 0 ? a : 0), (b > 0 ? a : 0))
