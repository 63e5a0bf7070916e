/**
    Fused optimizers for the HIP backend: drop-in replacements for $(D dopt.online.sgd), $(D dopt.online.adam) and
    $(D dopt.online.amsgrad) (same parameters, same $(D Updater) result).

    $(D dopt.online) appends the update rule to the graph as pointwise operations, with every scalar broadcast by a
    product with a ones vector.  That form runs on this backend unchanged, kernel by kernel.  The functions here
    compile only outputs, gradients and the projections that do not depend on the updated value, and apply the rule
    with ONE multi-tensor kernel of libdopthip.so that rounds once per node of that same expression tree: parameters
    and optimizer state come out identical to the graph form, bit for bit.

    Projections come in three kinds (online/sgd.d:75-85 applies them to the updated value inside its one plan):
    one that ignores the updated value (batch norm replaces its running statistics by outputs of the graph,
    nnet/layers/batchnorm.d:140-154) is computed by the step's plan and the kernel leaves that parameter alone; one
    that reads the updated value and nothing else the step computes (the operator-norm projections of
    nnet/lipschitz.d) runs as a second small plan after the kernel; one that also reads this batch's activations (the
    max-gain projections) can only be ordered correctly inside a single plan, so use $(D dopt.online) for those.

    Written where no D compiler exists: never compiled.
*/
module dopt.hip.online;

import std.algorithm : canFind, map;
import std.array : array;
import std.exception : enforce;

import dopt.core;
import dopt.hip;
import dopt.hip.shim;
import dopt.online : Projection, Updater;

private enum Rule
{
    sgd,
    adam,
    amsgrad
}

private class FusedUpdater
{
    this(Rule rule, Operation[] outputs, Operation[] wrt, Projection[Operation] projs)
    {
        mRule = rule;
        mOutputs = outputs.dup;

        auto grads = grad(outputs[0], wrt);
        auto stepNodes = topologicalSort(outputs);

        Operation[] planProj;       //projected values the step's plan computes itself
        Operation[] planProjTarget;
        Operation[] postProj;       //projections of the updated value, run after the kernel
        Operation[] postTarget;
        bool[] skip;

        foreach(w; wrt)
        {
            skip ~= false;

            if((w in projs) is null)
            {
                continue;
            }

            auto probe = float32(w.shape);
            auto projected = projs[w](probe);
            auto nodes = topologicalSort([projected]);

            if(!nodes.canFind!(x => x is probe))
            {
                planProj ~= projected;
                planProjTarget ~= w;
                skip[$ - 1] = true;
            }
            else
            {
                foreach(n; nodes)
                {
                    enforce(n is probe || n.opType != "variable" || !stepNodes.canFind!(x => x is n),
                        "a projection that reads both the updated value and other variables of the step cannot be " ~
                        "ordered by the fused updaters; use dopt.online for this model");
                }

                postProj ~= projs[w](w);
                postTarget ~= w;
            }
        }

        mPlan = new HIPPlan(outputs ~ grads ~ planProj, defaultPlanFlags);

        //Outputs are copied out, gradients are read in place, projected statistics go straight over their variables
        mRets = outputs.map!(x => allocate(x.volume * x.elementType.sizeOf)).array();
        mRets ~= new DeviceBuffer[grads.length];
        mRets ~= planProjTarget.map!(x => x.value).array();

        if(postProj.length != 0)
        {
            mPostPlan = new HIPPlan(postProj, defaultPlanFlags);
            mPostRets = postTarget.map!(x => x.value).array();
        }

        dopt_hip_tensor_ref[] refs;

        foreach(i, w; wrt)
        {
            auto wbuf = cast(HIPBuffer)w.value;
            enforce(wbuf !is null, "the fused updaters need parameters that live on the device (dopt.hip's allocator)");

            dopt_hip_tensor_ref r;
            r.w = cast(float *)wbuf.ptr;
            r.g = cast(const(float) *)mPlan.result(grads[i]).ptr;
            r.n = w.volume;
            r.skip_w = skip[i] ? 1 : 0;

            auto bytes = w.volume * float.sizeof;
            mState ~= HIPBuffer.create(bytes);
            r.m = cast(float *)mState[$ - 1].ptr;

            if(rule != Rule.sgd)
            {
                mState ~= HIPBuffer.create(bytes);
                r.v = cast(float *)mState[$ - 1].ptr;
            }

            if(rule == Rule.amsgrad)
            {
                mState ~= HIPBuffer.create(bytes);
                r.vhat = cast(float *)mState[$ - 1].ptr;
            }

            refs ~= r;
        }

        hipCheck(dopt_hip_optim_create(cast(int)refs.length, refs.ptr, &mHandle));
    }

    ~this()
    {
        if(mHandle !is null)
        {
            dopt_hip_optim_destroy(mHandle);
        }
    }

    DeviceBuffer[] update(DeviceBuffer[Operation] args)
    {
        //The plan reads the OLD parameters; the kernel then updates them in place
        mPlan.execute(args, mRets);

        final switch(mRule)
        {
            case Rule.sgd:
                hipCheck(dopt_hip_sgd_step(mHandle, scalar(mHyper[0]), scalar(mHyper[1]), mNesterov ? 1 : 0));
                break;

            case Rule.adam:
                hipCheck(dopt_hip_adam_step(mHandle, scalar(mHyper[0]), scalar(mHyper[1]), scalar(mHyper[2]),
                    scalar(mHyper[3]), &mB1, &mB2));
                break;

            case Rule.amsgrad:
                hipCheck(dopt_hip_amsgrad_step(mHandle, scalar(mHyper[0]), scalar(mHyper[1]), scalar(mHyper[2]),
                    scalar(mHyper[3]), &mB1, &mB2));
                break;
        }

        if(mPostPlan !is null)
        {
            mPostPlan.execute(null, mPostRets);
        }

        return mRets[0 .. mOutputs.length];
    }

    //Hyper-parameters are scalar Operations, as in dopt.online: their current value is read at every step
    static float scalar(Operation op)
    {
        return op.value.get!float[0];
    }

    Rule mRule;
    Operation[] mOutputs;
    Operation[] mHyper;
    bool mNesterov;
    float mB1 = 1.0f, mB2 = 1.0f;   //the running products beta^t of online/adam.d:44-46
    HIPPlan mPlan, mPostPlan;
    DeviceBuffer[] mRets, mPostRets;
    HIPBuffer[] mState;
    void *mHandle;
}

/**
    Stochastic gradient descent with momentum; see $(D dopt.online.sgd) (online/sgd.d:28-94) for the parameters.
*/
Updater sgd(Operation[] outputs, Operation[] wrt, Projection[Operation] projs,
    Operation learningRate = float32([], [0.01f]), Operation momentumRate = float32([], [0.0f]), bool nesterov = false)
{
    auto u = new FusedUpdater(Rule.sgd, outputs, wrt, projs);
    u.mHyper = [learningRate, momentumRate];
    u.mNesterov = nesterov;

    return &u.update;
}

/**
    ADAM; see $(D dopt.online.adam) (online/adam.d:32-93) for the parameters.
*/
Updater adam(Operation[] outputs, Operation[] wrt, Projection[Operation] projs,
    Operation alpha = float32([], [0.001f]), Operation beta1 = float32([], [0.9f]),
    Operation beta2 = float32([], [0.999f]), Operation eps = float32([], [1e-8]))
{
    auto u = new FusedUpdater(Rule.adam, outputs, wrt, projs);
    u.mHyper = [alpha, beta1, beta2, eps];

    return &u.update;
}

/**
    AMSGrad as the reference writes it (online/amsgrad.d:32-99): the step uses the new second moment, and the
    running maximum takes the OLD one.
*/
Updater amsgrad(Operation[] outputs, Operation[] wrt, Projection[Operation] projs,
    Operation alpha = float32([], [0.001f]), Operation beta1 = float32([], [0.9f]),
    Operation beta2 = float32([], [0.999f]), Operation eps = float32([], [1e-8]))
{
    auto u = new FusedUpdater(Rule.amsgrad, outputs, wrt, projs);
    u.mHyper = [alpha, beta1, beta2, eps];

    return &u.update;
}

///
unittest
{
    import std.random : uniform;

    //Fit y = 3x + 2, the scenario of the reference's own optimizer tests
    auto xdata = new float[100];
    auto ydata = new float[100];

    foreach(i; 0 .. 100)
    {
        xdata[i] = uniform(-10.0f, 10.0f);
        ydata[i] = 3.0f * xdata[i] + 2.0f;
    }

    auto x = float32([]);
    auto m = float32([]);
    auto c = float32([]);

    auto yhat = m * x + c;
    auto y = float32([]);

    auto loss = (yhat - y) * (yhat - y);

    auto updater = adam([loss], [m, c], null, float32([], [0.1f]));

    foreach(epoch; 0 .. 300)
    {
        foreach(i; 0 .. 100)
        {
            updater([
                x: buffer(xdata[i .. i + 1]),
                y: buffer(ydata[i .. i + 1])
            ]);
        }
    }

    import std.math : approxEqual;

    assert(approxEqual(m.value.get!float[0], 3.0f));
    assert(approxEqual(c.value.get!float[0], 2.0f));
}
