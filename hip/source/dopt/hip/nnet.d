/**
    HIP kernels for the neural-network operations (the counterpart of cuda/source/dopt/cuda/nnet/cudnn7.d):
    convolution and its two gradients, max pooling, softmax, ReLU, bias and batch normalisation.  Semantics are
    cuDNN's as the reference configures it: true convolution (filter flipped), NCHW / KCRS layouts, packed
    batch-norm outputs [y | mean | var] and [dx | dscale | dbias].

    Written where no D compiler exists: never compiled.
*/
module dopt.hip.nnet;

import dopt.core;
import dopt.hip;
import dopt.hip.shim;

package
{
    void initialize()
    {
        import std.functional : toDelegate;

        registerHIPKernel("convolution", toDelegate(&ctr!ConvolutionForward), true);
        registerHIPKernel("convolutionFeaturesGrad", toDelegate(&ctr!ConvolutionFeaturesGrad), true);
        registerHIPKernel("convolutionFiltersGrad", toDelegate(&ctr!ConvolutionFiltersGrad), true);
        registerHIPKernel("maxpool", toDelegate(&ctr!MaxpoolForward), true);
        registerHIPKernel("maxpoolGrad", toDelegate(&ctr!MaxpoolGrad), true);
        registerHIPKernel("softmax", toDelegate(&ctr!Softmax), true);
        registerHIPKernel("softmaxGrad", toDelegate(&ctr!SoftmaxGrad), true);
        registerHIPKernel("relu", toDelegate(&ctr!ReLU), true);
        registerHIPKernel("reluGrad", toDelegate(&ctr!ReLUGrad), true);
        registerHIPKernel("addBias", toDelegate(&ctr!AddBias), true);
        registerHIPKernel("addBiasGrad", toDelegate(&ctr!AddBiasGrad), true);
        registerHIPKernel("batchNormTrain", toDelegate(&ctr!BatchNormTrain), true);
        registerHIPKernel("batchNormGrad", toDelegate(&ctr!BatchNormGrad), true);
        registerHIPKernel("batchNormInference", toDelegate(&ctr!BatchNormInference), true);
    }
}

private
{
    HIPKernel ctr(K)(Operation op)
    {
        return new K(op);
    }

    const(float) *f(const(HIPBuffer) b)
    {
        return cast(const(float) *)b.ptr;
    }

    float *f(HIPBuffer b)
    {
        return cast(float *)b.ptr;
    }

    dopt_hip_conv_desc describe(const(size_t)[] x, const(size_t)[] w, size_t[] padding, size_t[] stride)
    {
        return dopt_hip_conv_desc(x[0], x[1], x[2], x[3], w[0], w[2], w[3], padding[0], padding[1], stride[0],
            stride[1]);
    }

    //[N, C, inner] of a tensor whose dimension 1 is the channel
    void nci(const(size_t)[] shape, out size_t n, out size_t c, out size_t inner)
    {
        n = shape[0];
        c = shape[1];
        inner = 1;

        foreach(s; shape[2 .. $])
        {
            inner *= s;
        }
    }

    class ConvolutionForward : HIPKernel
    {
        this(Operation op)
        {
            mDesc = describe(op.deps[0].shape, op.deps[1].shape, op.attributes["padding"].get!(size_t[]),
                op.attributes["stride"].get!(size_t[]));
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_conv_fwd(&mDesc, f(inputs[0]), f(inputs[1]), f(output)));
        }

        dopt_hip_conv_desc mDesc;
    }

    class ConvolutionFeaturesGrad : HIPKernel
    {
        this(Operation op)
        {
            //deps: the gradient of the output, the filters; the features' shape is an attribute
            mDesc = describe(op.attributes["featuresShape"].get!(size_t[]), op.deps[1].shape,
                op.attributes["padding"].get!(size_t[]), op.attributes["stride"].get!(size_t[]));
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_conv_bwd_data(&mDesc, f(inputs[0]), f(inputs[1]), f(output)));
        }

        dopt_hip_conv_desc mDesc;
    }

    class ConvolutionFiltersGrad : HIPKernel
    {
        this(Operation op)
        {
            //deps: the gradient of the output, the features; the filters' shape is an attribute
            mDesc = describe(op.deps[1].shape, op.attributes["filtersShape"].get!(size_t[]),
                op.attributes["padding"].get!(size_t[]), op.attributes["stride"].get!(size_t[]));
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_conv_bwd_filter(&mDesc, f(inputs[0]), f(inputs[1]), f(output)));
        }

        dopt_hip_conv_desc mDesc;
    }

    class MaxpoolForward : HIPKernel
    {
        this(Operation op)
        {
            mShape = op.deps[0].shape.dup;
            mDims = op.attributes["dims"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_maxpool_fwd(mShape[0], mShape[1], mShape[2], mShape[3], mDims[0], mDims[1], f(inputs[0]),
                f(output)));
        }

        size_t[] mShape, mDims;
    }

    class MaxpoolGrad : HIPKernel
    {
        this(Operation op)
        {
            mShape = op.attributes["featuresShape"].get!(size_t[]).dup;
            mDims = op.attributes["dims"].get!(size_t[]).dup;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: dy, y, x.  The pooled values are recomputed from x, so y is not read.
            hipCheck(dopt_hip_maxpool_bwd(mShape[0], mShape[1], mShape[2], mShape[3], mDims[0], mDims[1], f(inputs[0]),
                f(inputs[2]), f(output)));
        }

        size_t[] mShape, mDims;
    }

    class Softmax : HIPKernel
    {
        this(Operation op)
        {
            nci(op.shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_softmax_fwd(mN, mC, mInner, f(inputs[0]), f(output)));
        }

        size_t mN, mC, mInner;
    }

    class SoftmaxGrad : HIPKernel
    {
        this(Operation op)
        {
            nci(op.shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: dy, y
            hipCheck(dopt_hip_softmax_bwd(mN, mC, mInner, f(inputs[0]), f(inputs[1]), f(output)));
        }

        size_t mN, mC, mInner;
    }

    class ReLU : HIPKernel
    {
        this(Operation op)
        {
            mVolume = op.volume;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_relu_fwd(mVolume, f(inputs[0]), f(output)));
        }

        size_t mVolume;
    }

    class ReLUGrad : HIPKernel
    {
        this(Operation op)
        {
            mVolume = op.volume;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: dy, y, x.  dx = x > 0 ? dy : 0
            hipCheck(dopt_hip_relu_bwd(mVolume, f(inputs[0]), f(inputs[2]), f(output)));
        }

        size_t mVolume;
    }

    class AddBias : HIPKernel
    {
        this(Operation op)
        {
            nci(op.shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            hipCheck(dopt_hip_bias_fwd(mN, mC, mInner, f(inputs[0]), f(inputs[1]), f(output)));
        }

        size_t mN, mC, mInner;
    }

    class AddBiasGrad : HIPKernel
    {
        this(Operation op)
        {
            nci(op.deps[0].shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //The plain sum over batch and positions.  (The reference passes beta = 1 to cuDNN and so adds to what the
            //output buffer held; the two agree on a plan's first execution.)
            hipCheck(dopt_hip_bias_bwd(mN, mC, mInner, f(inputs[0]), f(output)));
        }

        size_t mN, mC, mInner;
    }

    class BatchNormTrain : HIPKernel
    {
        this(Operation op)
        {
            nci(op.deps[0].shape, mN, mC, mInner);
            mMomentum = op.attributes["momentum"].get!double;
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: x, scale, bias, running mean, running variance; output [y | new mean | new variance]
            hipCheck(dopt_hip_bn_train(mN, mC, mInner, mMomentum, f(inputs[0]), f(inputs[1]), f(inputs[2]), f(inputs[3]),
                f(inputs[4]), f(output)));
        }

        size_t mN, mC, mInner;
        double mMomentum;
    }

    class BatchNormGrad : HIPKernel
    {
        this(Operation op)
        {
            nci(op.deps[1].shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: dy, x, scale; output [dx | dscale | dbias] at the front of a buffer the judge sizes generously
            hipCheck(dopt_hip_bn_grad(mN, mC, mInner, f(inputs[0]), f(inputs[1]), f(inputs[2]), f(output)));
        }

        size_t mN, mC, mInner;
    }

    class BatchNormInference : HIPKernel
    {
        this(Operation op)
        {
            nci(op.deps[0].shape, mN, mC, mInner);
        }

        override void execute(const(HIPBuffer)[] inputs, HIPBuffer output)
        {
            //deps: x, scale, bias, mean, variance
            hipCheck(dopt_hip_bn_infer(mN, mC, mInner, f(inputs[0]), f(inputs[1]), f(inputs[2]), f(inputs[3]),
                f(inputs[4]), f(output)));
        }

        size_t mN, mC, mInner;
    }
}

unittest
{
    //core/ops/nnet.d: a true convolution (the filter is flipped)
    auto features = float32([1, 1, 3, 5], [
        1.0f, 1.0f, 1.0f, 0.0f, 0.0f,
        1.0f, 1.0f, 1.0f, 0.0f, 0.0f,
        1.0f, 1.0f, 1.0f, 0.0f, 0.0f
    ]);

    auto filters = float32([1, 1, 1, 2], [-1.0f, 1.0f]);
    auto result = convolution(features, filters);

    assert(evaluateHIP(result).get!float == [0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 0.0f, 1.0f, 0.0f]);
}
