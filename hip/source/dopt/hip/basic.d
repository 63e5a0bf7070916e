/**
    HIP kernels for the layout operations: slice, pad, repeat, transpose (the counterpart of
    cuda/source/dopt/cuda/basic.d).  Each kernel object reads shapes and attributes off its Operation once and makes
    one call into libdopthip.so per execution.

    Written where no D compiler exists: never compiled.
*/
module dopt.hip.basic;

import dopt.core;
import dopt.hip;
import dopt.hip.shim;

package
{
    void initialize()
    {
        import std.functional : toDelegate;

        registerHIPKernel("slice", toDelegate(&hipKernelCtr!Slice), true);
        registerHIPKernel("pad", toDelegate(&hipKernelCtr!Pad), true);
        registerHIPKernel("repeat", toDelegate(&hipKernelCtr!Repeat), true);
        registerHIPKernel("transpose", toDelegate(&hipKernelCtr!Transpose), true);
    }

    HIPKernel hipKernelCtr(K)(Operation op)
    {
        return new K(op);
    }
}

private
{
    class Slice : HIPKernel
    {
        this(Operation op)
        {
            mInShape = op.deps[0].shape.dup;
            mOutShape = op.shape.dup;
            mStart = op.attributes["start"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_slice(cast(int)mInShape.length, mInShape.ptr, mOutShape.ptr, mStart.ptr,
                inputs[0].ptr, output.ptr));
        }

        size_t[] mInShape, mOutShape, mStart;
    }

    class Pad : HIPKernel
    {
        this(Operation op)
        {
            mInShape = op.deps[0].shape.dup;
            mOutShape = op.shape.dup;
            mBefore = op.attributes["before"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //One kernel writes every element of the output, zeros included
            hipCheck(dopt_hip_pad(cast(int)mInShape.length, mInShape.ptr, mOutShape.ptr, mBefore.ptr,
                inputs[0].ptr, output.ptr));
        }

        size_t[] mInShape, mOutShape, mBefore;
    }

    class Repeat : HIPKernel
    {
        this(Operation op)
        {
            mInShape = op.deps[0].shape.dup;
            mReps = op.attributes["repetitions"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_repeat(cast(int)mInShape.length, mInShape.ptr, mReps.ptr, inputs[0].ptr, output.ptr));
        }

        size_t[] mInShape, mReps;
    }

    class Transpose : HIPKernel
    {
        this(Operation op)
        {
            import std.exception : enforce;

            auto order = op.attributes["order"].get!(size_t[]);
            auto shape = op.deps[0].shape;

            mIdentity = true;

            foreach(i, o; order)
            {
                mIdentity = mIdentity && o == i;
            }

            //Like the CUDA backend (one cublasSgeam call), only matrices are transposed on the device
            enforce(mIdentity || shape.length == 2, "transpose is only implemented for rank 2 tensors");

            mVolume = op.volume;

            if(shape.length == 2)
            {
                mRows = shape[0];
                mCols = shape[1];
            }
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            if(mIdentity)
            {
                hipCheck(dopt_hip_copy_d2d(output.ptr, inputs[0].ptr, mVolume * 4));
            }
            else
            {
                hipCheck(dopt_hip_transpose2d(mRows, mCols, inputs[0].ptr, output.ptr));
            }
        }

        bool mIdentity;
        size_t mRows, mCols, mVolume;
    }
}

unittest
{
    auto a = int32([3, 3], [1, 2, 3, 4, 5, 6, 7, 8, 9]).slice([1, 1], [3, 3]);

    assert(evaluateHIP(a).get!int == [5, 6, 8, 9]);
}
