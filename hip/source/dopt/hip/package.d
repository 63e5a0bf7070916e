/**
    The dopt HIP backend for AMD MI355X (gfx950): the counterpart of $(D dopt.cuda) over libdopthip.so.

    Same plugin surface as the CUDA backend (cuda/source/dopt/cuda/package.d), with HIP for CUDA in every name:
    $(D HIPKernel), $(D HIPKernelCtr), $(D HIPBuffer), $(D HIPPlan), $(D evaluateHIP), $(D registerHIPKernel),
    $(D deregisterHIPKernel), $(D listHIPOperations).  Importing this module installs the backend as dopt's default
    evaluator, compiler and variable allocator, exactly as importing $(D dopt.cuda) does.

    There is one plan class.  $(D HIPPlan) hands the whole graph to the planner inside libdopthip.so
    (include/dopt_hip_plan.h), which owns the topological order, the per-operation buffers and the kernel objects and
    can apply its rewrites (views, fused pairs, pointwise chains, graph replay).  The kernel classes of
    dopt.hip.basic / math / nnet / random each make one call into the kernel library; they exist so that D code can
    construct and run a single kernel the way it does with $(D dopt.cuda), and so that the D registry lists every
    operation.  Kernels registered from D take part in plans too: the planner calls them back through a C trampoline.

    Written where no D compiler exists (the library's build image has none): this package has never been compiled.

    Authors: the dopt.hip contributors
*/
module dopt.hip;

import std.conv : to;
import std.exception : enforce;
import std.string : fromStringz, toStringz;
import std.variant : Variant;

import dopt.core;
import dopt.hip.shim;

static import dopt.hip.basic;
static import dopt.hip.math;
static import dopt.hip.nnet;
static import dopt.hip.random;

alias HIPKernelCtr = HIPKernel delegate(Operation op);

/// Rewrites the native planner applies unless told otherwise; see include/dopt_hip_plan.h.
__gshared uint defaultPlanFlags = DOPT_HIP_PLAN_VIEWS | DOPT_HIP_PLAN_FUSE;

/**
    Turns a status code of the library into the exception the reference raises with $(D enforce).
*/
void hipCheck(int rc, string file = __FILE__, size_t line = __LINE__)
{
    if(rc != 0)
    {
        throw new Exception(dopt_hip_last_error().fromStringz.idup, file, line);
    }
}

package int hipType(DataType t)
{
    switch(t)
    {
        case DataType.float32:
            return DOPT_HIP_F32;

        case DataType.int32:
            return DOPT_HIP_I32;

        default:
            throw new Exception("Element type not supported.");
    }
}

/**
    Registers all the kernels of the HIP backend and makes it dopt's default backend.
*/
shared static this()
{
    try
    {
        hipCheck(dopt_hip_init(0));

        dopt.hip.basic.initialize();
        dopt.hip.math.initialize();
        dopt.hip.nnet.initialize();
        dopt.hip.random.initialize();

        import std.functional : toDelegate;
        defaultEvaluator = toDelegate(&evaluateHIP);
        defaultCompiler = (Operation[] ops)
        {
            return cast(Plan)new HIPPlan(ops, defaultPlanFlags);
        };
        defaultVarAllocator = (size_t numBytes) { return cast(DeviceBuffer)HIPBuffer.create(numBytes); };
    }
    catch(Exception e)
    {
        //No usable device: dopt keeps whatever backend was installed before (the CPU one), as with dopt.cuda
    }
}

/**
    Provides a common interface for HIP kernels.
*/
interface HIPKernel
{
    /**
        Runs the kernel with the given inputs and outputs.

        Params:
            inputs = One buffer per dependency of the operation used to construct this kernel, in order.
            output = The destination buffer.
    */
    void execute(const(HIPBuffer)[] inputs, HIPBuffer output);
}

/**
    Device memory from the library's pooled allocator.
*/
class HIPBuffer : DeviceBuffer
{
    public
    {
        /**
            Allocates numBytes of zero-filled device memory.  A request for zero bytes yields an empty buffer.
        */
        static HIPBuffer create(size_t numBytes)
        {
            auto ret = new HIPBuffer();

            if(numBytes == 0)
            {
                return ret;
            }

            ret.mNumBytes = numBytes;
            ret.mOwned = true;
            hipCheck(dopt_hip_malloc(&ret.mPtr, numBytes));

            return ret;
        }

        /**
            A buffer object over device memory that someone else owns (a plan's result, a caller's staging area).
        */
        static HIPBuffer view(void *ptr, size_t numBytes)
        {
            auto ret = new HIPBuffer();
            ret.mPtr = ptr;
            ret.mNumBytes = numBytes;

            return ret;
        }

        /**
            Returns the memory of buf to the pool.
        */
        static void destroy(HIPBuffer buf)
        {
            if(buf.mOwned && buf.mPtr !is null)
            {
                hipCheck(dopt_hip_free(buf.mPtr));
                buf.mPtr = null;
            }
        }

        ~this()
        {
            //The pool is guarded against a finaliser thread; errors cannot be thrown from here
            if(mOwned && mPtr !is null)
            {
                dopt_hip_free(mPtr);
            }
        }

        override void set(const void[] buf)
        {
            enforce(buf.length == mNumBytes, "input buffer is the wrong length.");
            hipCheck(dopt_hip_copy_h2d(mPtr, buf.ptr, buf.length));
        }

        override void set(const DeviceBuffer buf)
        {
            import dopt.cpu : CPUBuffer;

            enforce(numBytes == buf.numBytes, "Mismatch in buffer size");

            auto hipbuf = cast(HIPBuffer)buf;
            auto cpubuf = cast(CPUBuffer)buf;

            if(hipbuf !is null)
            {
                hipCheck(dopt_hip_copy_d2d(mPtr, hipbuf.ptr, numBytes));
            }
            else if(cpubuf !is null)
            {
                hipCheck(dopt_hip_copy_h2d(mPtr, cpubuf.raw.ptr, numBytes));
            }
            else
            {
                super.set(buf);
            }
        }

        override void get(void[] buf) const
        {
            enforce(buf.length == mNumBytes, "output buffer is the wrong length.");
            hipCheck(dopt_hip_copy_d2h(buf.ptr, mPtr, buf.length));
        }

        override size_t numBytes() const
        {
            return mNumBytes;
        }

        /// The device pointer.
        inout(void) *ptr() inout
        {
            return mPtr;
        }
    }

    private
    {
        size_t mNumBytes;
        void *mPtr;
        bool mOwned;

        this()
        {
            //
        }
    }
}

/**
    A plan executed by the planner inside libdopthip.so: the graph is handed over once, operation by operation
    (type, judged output type, dependencies, attributes), and executions are one call each.
*/
class HIPPlan : Plan
{
    public
    {
        this(Operation[] outputs, uint flags = defaultPlanFlags)
        {
            import std.array : array;

            super(outputs);

            hipCheck(dopt_hip_graph_create(&mGraph));

            foreach(o; topologicalSort(outputs))
            {
                int[] deps;

                foreach(d; o.deps)
                {
                    deps ~= mIds[d];
                }

                auto shape = o.shape.dup;
                int id;
                hipCheck(dopt_hip_graph_add_op(mGraph, o.opType.toStringz, hipType(o.elementType), cast(int)shape.length,
                    shape.ptr, cast(int)deps.length, deps.ptr, &id));
                mIds[o] = id;

                foreach(key, val; o.attributes)
                {
                    setAttribute(id, key, val);
                }

                if(o.opType == "variable")
                {
                    mVariables ~= o;
                }
                else if(o.opType == "constant")
                {
                    void *ptr;
                    size_t bytes;
                    hipCheck(dopt_hip_graph_value(mGraph, id, &ptr, &bytes));
                    HIPBuffer.view(ptr, bytes).set(o.value);
                }
            }

            int[] outIds;

            foreach(o; mOutputs)
            {
                outIds ~= mIds[o];
            }

            //Kernels registered from D are constructed by the planner through ctorTrampoline, which needs to find
            //the Operation behind an id
            tlsBuilding = this;
            scope(exit) tlsBuilding = null;

            foreach(o, id; mIds)
            {
                mOpOfId[id] = o;
            }

            hipCheck(dopt_hip_plan_create(mGraph, cast(int)outIds.length, outIds.ptr, flags, &mPlan));
        }

        ~this()
        {
            cleanup();
        }

        void cleanup()
        {
            if(mPlan !is null)
            {
                dopt_hip_plan_destroy(mPlan);
                mPlan = null;
            }

            if(mGraph !is null)
            {
                dopt_hip_graph_destroy(mGraph);
                mGraph = null;
            }
        }

        /**
            The plan-owned device buffer that holds the value of op after an execution (valid until cleanup).
        */
        HIPBuffer result(Operation op)
        {
            void *ptr;
            size_t bytes;
            hipCheck(dopt_hip_plan_result(mPlan, mIds[op], &ptr, &bytes));

            return HIPBuffer.view(ptr, bytes);
        }

        /**
            Accumulated device microseconds per operation type (needs DOPT_HIP_PLAN_TIMING in the flags).
        */
        long[string] profiler()
        {
            import std.algorithm : splitter;
            import std.array : split;

            long[string] ret;
            size_t needed;
            hipCheck(dopt_hip_plan_profile(mPlan, null, 0, &needed));
            auto buf = new char[needed];
            hipCheck(dopt_hip_plan_profile(mPlan, buf.ptr, buf.length, null));

            foreach(line; buf.ptr.fromStringz.splitter('\n'))
            {
                auto fields = line.split(' ');

                if(fields.length == 3)
                {
                    ret[fields[0].idup] = cast(long)fields[1].to!double;
                }
            }

            return ret;
        }
    }

    protected
    {
        override void executeImpl(DeviceBuffer[Operation] args, DeviceBuffer[] rets)
        {
            foreach(o; args.keys)
            {
                enforce(o.opType == "variable",
                    "All assignments in args must be for Operations with an opType of 'variable'");
            }

            //Every variable of the graph is bound on every execution: to the caller's buffer when there is one,
            //to the variable's own value otherwise (cuda/package.d:367-401)
            int[] argOps;
            const(void)*[] argPtrs;
            int[] argOnHost;
            ubyte[][] keepAlive;

            foreach(v; mVariables)
            {
                import dopt.cpu : CPUBuffer;

                DeviceBuffer given = (v in args) ? args[v] : v.value;
                enforce(given.numBytes == v.volume * v.elementType.sizeOf, "Mismatch in buffer size");

                argOps ~= mIds[v];

                if(auto hipbuf = cast(HIPBuffer)given)
                {
                    argPtrs ~= hipbuf.ptr;
                    argOnHost ~= 0;
                }
                else if(auto cpubuf = cast(CPUBuffer)given)
                {
                    argPtrs ~= cpubuf.raw.ptr;
                    argOnHost ~= 1;
                }
                else
                {
                    keepAlive ~= given.get!ubyte();
                    argPtrs ~= keepAlive[$ - 1].ptr;
                    argOnHost ~= 1;
                }
            }

            void*[] retPtrs;
            HIPBuffer[] staged = new HIPBuffer[rets.length];

            foreach(i, r; rets)
            {
                if(r is null)
                {
                    retPtrs ~= null;       //the caller reads this output in place (resultPtr): no copy
                }
                else if(auto hipbuf = cast(HIPBuffer)r)
                {
                    retPtrs ~= hipbuf.ptr;
                }
                else
                {
                    staged[i] = HIPBuffer.create(r.numBytes);
                    retPtrs ~= staged[i].ptr;
                }
            }

            hipCheck(dopt_hip_plan_execute(mPlan, cast(int)argOps.length, argOps.ptr, argPtrs.ptr, argOnHost.ptr,
                cast(int)retPtrs.length, retPtrs.ptr));

            foreach(i, r; rets)
            {
                if(staged[i] !is null)
                {
                    r.set(staged[i]);
                    HIPBuffer.destroy(staged[i]);
                }
            }
        }
    }

    private
    {
        void *mGraph;
        void *mPlan;
        int[Operation] mIds;
        Operation[int] mOpOfId;
        Operation[] mVariables;

        void setAttribute(int id, string key, Variant val)
        {
            if(val.type == typeid(size_t[]))
            {
                auto v = val.get!(size_t[]);
                hipCheck(dopt_hip_graph_set_attr_sizes(mGraph, id, key.toStringz, v.ptr, cast(int)v.length));
            }
            else if(val.type == typeid(size_t))
            {
                size_t v = val.get!size_t;
                hipCheck(dopt_hip_graph_set_attr_sizes(mGraph, id, key.toStringz, &v, 1));
            }
            else if(val.type == typeid(double))
            {
                hipCheck(dopt_hip_graph_set_attr_double(mGraph, id, key.toStringz, val.get!double));
            }
            else if(val.type == typeid(float))
            {
                hipCheck(dopt_hip_graph_set_attr_double(mGraph, id, key.toStringz, cast(double)val.get!float));
            }
            //Anything else is not a payload a kernel reads (the "type" of variables and constants is passed above)
        }
    }
}

/// Kept for code written against the earlier name of the plan class.
alias NativeHIPPlan = HIPPlan;

/**
    Used for performing a one-off evaluation of a set of operations.

    Params:
        ops = The operations to be evaluated.
        args = A set of optional variable assignments.

    Returns:
        The result of evaluating $(D ops).
*/
DeviceBuffer[] evaluateHIP(Operation[] ops, DeviceBuffer[Operation] args = null)
{
    Plan p = new HIPPlan(ops, 0);

    return p.execute(args);
}

/// ditto
DeviceBuffer evaluateHIP(Operation op, DeviceBuffer[Operation] args = null)
{
    return evaluateHIP([op], args)[0];
}

/**
    Registers a HIP kernel constructor for a given operation type.

    Params:
        opName = The type of operation this kernel constructor caters to.
        kernelCtr = The constructor that should be associated with operations with the type $(D opType).
        native = Set by the backend's own modules: the library already has a kernel of this name built in, so
                 only the D registry needs to know it.
*/
void registerHIPKernel(string opName, HIPKernelCtr kernelCtr, bool native = false)
{
    enforce((opName in mKernelCtrs) is null,
        "A HIPKernelCtr is already registered for the operation '" ~ opName ~ "'");

    if(!native)
    {
        //The planner inside the library calls back into D for this operation
        mUserCtrs ~= kernelCtr;
        hipCheck(dopt_hip_register_kernel(opName.toStringz, &ctorTrampoline, cast(void *)(mUserCtrs.length - 1)));
    }

    mKernelCtrs[opName] = kernelCtr;
}

/**
    Deregisters a kernel constructor associated with the given operation type.
*/
void deregisterHIPKernel(string opType)
{
    mKernelCtrs.remove(opType);
    hipCheck(dopt_hip_deregister_kernel(opType.toStringz));
}

/**
    Provides a list of all operation types supported by the HIP backend.
*/
string[] listHIPOperations()
{
    return mKernelCtrs.keys ~ ["variable", "reshape"];
}

private
{
    HIPKernelCtr[string] mKernelCtrs;
    HIPKernelCtr[] mUserCtrs;
    HIPPlan tlsBuilding;

    //A D kernel object kept alive for the planner, and the buffers it is handed on each execution
    class Trampolined
    {
        HIPKernel kernel;
    }

    Trampolined[] mTrampolined;

    extern(C) int ctorTrampoline(void *graph, int op, void *user, dopt_hip_kernel *result) nothrow
    {
        try
        {
            auto plan = tlsBuilding;

            if(plan is null || (op in plan.mOpOfId) is null)
            {
                return 1;
            }

            auto t = new Trampolined();
            t.kernel = mUserCtrs[cast(size_t)user](plan.mOpOfId[op]);

            if(t.kernel is null)
            {
                return 1;
            }

            mTrampolined ~= t;     //the garbage collector must not reclaim what only C code points to
            result.self = cast(void *)t;
            result.execute = &executeTrampoline;
            result.destroy = null;

            return 0;
        }
        catch(Exception e)
        {
            return 1;
        }
    }

    extern(C) int executeTrampoline(void *self, int ninputs, const(const(void)*)* inputs, const(size_t)* inputBytes,
        void *output, size_t outputBytes) nothrow
    {
        try
        {
            auto t = cast(Trampolined)self;
            HIPBuffer[] bufs;

            foreach(i; 0 .. ninputs)
            {
                bufs ~= HIPBuffer.view(cast(void *)inputs[i], inputBytes[i]);
            }

            t.kernel.execute(bufs, HIPBuffer.view(output, outputBytes));

            return 0;
        }
        catch(Exception e)
        {
            return 2;
        }
    }
}

unittest
{
    auto a = float32([], [3.0f]);
    auto b = float32([], [4.0f]);
    auto c = float32([], [-1.0f]);

    auto y = a * b + c;

    assert(evaluateHIP(y).get!float[0] == 11.0f);
}
