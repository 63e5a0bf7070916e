/**
    The `uniform` operation on the device (the counterpart of cuda/source/dopt/cuda/random.d): a counter-based
    Philox4x32-10 kernel.  A kernel object draws its seed once, like the reference's generator, and numbers its
    executions, so that every evaluation yields fresh values from (0, 1].

    Written where no D compiler exists: never compiled.
*/
module dopt.hip.random;

import dopt.core;
import dopt.hip;
import dopt.hip.shim;

package
{
    void initialize()
    {
        registerHIPKernel("uniform", (Operation op) { return cast(HIPKernel)new Uniform(op); }, true);
    }
}

private
{
    class Uniform : HIPKernel
    {
        this(Operation op)
        {
            import std.random : unpredictableSeed;

            mVolume = op.volume;
            mSeed = (cast(ulong)unpredictableSeed << 32) | unpredictableSeed;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_uniform(mSeed, mCall++, mVolume, cast(float *)output.ptr));
        }

        size_t mVolume;
        ulong mSeed, mCall;
    }
}
