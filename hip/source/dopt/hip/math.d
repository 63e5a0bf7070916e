/**
    HIP kernels for the pointwise operations, matmul and the reductions (the counterpart of
    cuda/source/dopt/cuda/math.d).  Pointwise kernels are instantiated at run time by the library (hipRTC templates,
    one per operation and element type); sum, maxElement and argmin, which the CUDA backend sends on a round trip
    through the CPU evaluator, run on the device.

    Written where no D compiler exists: never compiled.
*/
module dopt.hip.math;

import std.string : toStringz;

import dopt.core;
import dopt.hip;
import dopt.hip.shim;

package
{
    void initialize()
    {
        //Binary and unary pointwise operations: the names dopt_hip_pointwise accepts
        static immutable string[] binary = ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq",
            "max", "min", "pow"];
        static immutable string[] unary = ["neg", "abs", "sgn", "exp", "log", "sqrt", "sin", "cos", "tan", "asin",
            "acos", "atan", "sinh", "cosh", "tanh", "asinh", "acosh", "atanh"];

        foreach(name; binary)
        {
            registerHIPKernel(name, pointwiseCtr(name, 2), true);
        }

        foreach(name; unary)
        {
            registerHIPKernel(name, pointwiseCtr(name, 1), true);
        }

        //ops/math.d lists atan2 with the unary functions; it takes two operands where the graph supplies them
        registerHIPKernel("atan2", (Operation op) { return cast(HIPKernel)new Pointwise(op, "atan2", op.deps.length == 2 ? 2 : 1); },
            true);

        registerHIPKernel("matmul", (Operation op) { return cast(HIPKernel)new Matmul(op); }, true);
        registerHIPKernel("sum", (Operation op) { return cast(HIPKernel)new Reduce(op, "sum"); }, true);
        registerHIPKernel("maxElement", (Operation op) { return cast(HIPKernel)new Reduce(op, "maxElement"); }, true);
        registerHIPKernel("argmin", (Operation op) { return cast(HIPKernel)new Argmin(op); }, true);
    }
}

private
{
    HIPKernelCtr pointwiseCtr(string name, int arity)
    {
        return (Operation op) { return cast(HIPKernel)new Pointwise(op, name, arity); };
    }

    class Pointwise : HIPKernel
    {
        this(Operation op, string name, int arity)
        {
            mName = name.toStringz;
            mArity = arity;
            mType = hipType(op.elementType);
            mVolume = op.volume;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_pointwise(mName, mType, mVolume, inputs[0].ptr, mArity == 2 ? inputs[1].ptr : null,
                output.ptr));
        }

        immutable(char) *mName;
        int mArity, mType;
        size_t mVolume;
    }

    class Matmul : HIPKernel
    {
        this(Operation op)
        {
            import std.exception : enforce;

            enforce(op.elementType == DataType.float32, "Element type not supported.");

            mM = op.deps[0].shape[0];
            mK = op.deps[0].shape[1];
            mN = op.deps[1].shape[1];
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //Row-major C = A * B; no operand swap is needed, the library is row-major throughout
            hipCheck(dopt_hip_sgemm(mM, mN, mK, cast(const(float) *)inputs[0].ptr, cast(const(float) *)inputs[1].ptr,
                cast(float *)output.ptr));
        }

        size_t mM, mN, mK;
    }

    class Reduce : HIPKernel
    {
        this(Operation op, string name)
        {
            mName = name.toStringz;
            mType = hipType(op.elementType);
            mShape = op.deps[0].shape.dup;
            mAxes = op.attributes["axes"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_reduce(mName, mType, mShape.ptr, cast(int)mShape.length, mAxes.ptr, cast(int)mAxes.length,
                inputs[0].ptr, output.ptr));
        }

        immutable(char) *mName;
        int mType;
        size_t[] mShape, mAxes;
    }

    class Argmin : HIPKernel
    {
        this(Operation op)
        {
            mType = hipType(op.deps[0].elementType);
            mShape = op.deps[0].shape.dup;
            mAxis = op.attributes["axis"].get!size_t;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_argmin(mType, mShape.ptr, cast(int)mShape.length, mAxis, inputs[0].ptr,
                cast(int *)output.ptr));
        }

        int mType;
        size_t[] mShape;
        size_t mAxis;
    }
}

unittest
{
    auto a = float32([2, 3], [1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f]);
    auto b = float32([3, 2], [1.0f, 0.0f, 0.0f, 1.0f, 1.0f, 1.0f]);

    assert(evaluateHIP(matmul(a, b)).get!float == [4.0f, 5.0f, 10.0f, 11.0f]);
}
