// Moves every connected region of hip operators out of the stackvm functions into a function of module kind
// "hip", so that the kmodel gets a hip module whose functions the stackvm code reaches through EXTCALL
// (src/Native/src/runtime/stackvm/ops/control.cpp:25-75).
//
// A region is a set of hip calls that read one outside activation X (any number of times: a residual add
// may take X itself) and otherwise only each other; the calls of a network between its Quantize and its
// Dequantize usually form one region.  Calls are visited in dependency order and each joins the region of its
// producers when all of its activations are that region's members or its X; regions that read the same X
// merge.  A call that would need a second outside activation cannot be a one-input function: it goes back to
// the neutral operators it was lowered from (IHipOp.Raise) and runs on the stackvm kernels.
//
// A region becomes
//   PrimFunction("hip_<n>", "hip", Sequential(HipStore(value_0, out_0), ...), in, out_0, ...)
//   PrimFunctionWrapper(that, 1)
// both added to the module (ModelBuilder groups functions by ModuleKind,
// src/Nncase.CodeGen/CodeGen/ModelBuilder.cs:39-46), and each value used outside the region becomes
// Call(wrapper, X) or GetItem(Call(wrapper, X), k).  This is the form the stackvm code generator already emits
// as "LdFunctionId ; EXTCALL 1, true" without a change
// (modules/Nncase.Modules.StackVM/CodeGen/StackVM/CodegenVisitor.cs:306-310); at run time EXTCALL allocates the
// outputs from the function's parameter types and passes them behind the input (control.cpp:50-68).
using System;
using System.Collections.Generic;
using System.Linq;
using System.Threading.Tasks;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.Runtime.Hip;
using Nncase.TIR;
using Nncase.Utilities;

namespace Nncase.Passes;

public sealed class OutlineHipFunctionsPass : ModulePass
{
    private int _count;

    /// <summary>The activations of a hip call: its leading arguments, with the tuple of a HipQConcat opened.</summary>
    public static IEnumerable<Expr> Activations(Call call)
    {
        var op = (IHipOp)call.Target;
        for (int i = 0; i < op.Activations; i++)
        {
            if (call.Arguments[i] is IR.Tuple tuple)
            {
                foreach (var field in tuple.Fields.ToArray())
                {
                    yield return field;
                }
            }
            else
            {
                yield return call.Arguments[i];
            }
        }
    }

    protected override Task<IRModule> RunCoreAsync(IRModule module, RunPassContext context)
    {
        foreach (var function in module.Functions.OfType<Function>().ToArray())
        {
            var calls = new List<Call>();
            new HipCalls(calls).Visit(function.Body);
            var regionOf = new Dictionary<Call, Region>(ReferenceEqualityComparer.Instance);
            var regions = new List<Region>();
            foreach (var call in calls)
            {
                var region = Assign(call, regionOf, regions);
                if (region is null)
                {
                    var raised = ((IHipOp)call.Target).Raise(call.Arguments.ToArray());
                    CompilerServices.InferenceType(raised);
                    ReplaceUtility.ReplaceAllUsesWith(call, raised);
                }
                else
                {
                    region.Members.Add(call);
                    regionOf[call] = region;
                }
            }

            foreach (var region in regions.Where(r => r.Members.Count > 0))
            {
                Outline(module, function, region);
            }
        }

        return Task.FromResult(module);
    }

    private static bool IsHipCall(Expr expr) => expr is Call { Target: IHipOp };

    // the region `call` belongs to, a new one, or null when it cannot be part of a one-input function
    private static Region? Assign(Call call, Dictionary<Call, Region> regionOf, List<Region> regions)
    {
        var inside = new List<Region>();
        var outside = new List<Expr>();
        foreach (var activation in Activations(call))
        {
            if (activation is Call producer && regionOf.TryGetValue(producer, out var r))
            {
                if (!inside.Contains(r.Root))
                {
                    inside.Add(r.Root);
                }
            }
            else if (!outside.Any(e => ReferenceEquals(e, activation)))
            {
                outside.Add(activation);
            }
        }

        if (inside.Count == 0)
        {
            if (outside.Count != 1)
            {
                return null;
            }

            var region = new Region(outside[0]);
            regions.Add(region);
            return region;
        }

        var input = inside[0].Input;
        if (inside.Any(r => !ReferenceEquals(r.Input, input)) || outside.Any(e => !ReferenceEquals(e, input)))
        {
            return null;
        }

        // regions that read the same X and meet in this call become one (members stay in visiting order)
        foreach (var other in inside.Skip(1))
        {
            inside[0].Members.AddRange(other.Members);
            other.Members.Clear();
            other.MergedInto = inside[0];
        }

        return inside[0];
    }

    private void Outline(IRModule module, Function function, Region region)
    {
        var members = new HashSet<Expr>(region.Members, ReferenceEqualityComparer.Instance);

        // a value leaves the region when something other than a member (or a member's tuple) reads it
        bool Leaves(Call value) => ReferenceEquals(function.Body, value) || value.Users.Any(u =>
            u is IR.Tuple tuple ? (ReferenceEquals(function.Body, tuple) || tuple.Users.Any(tu => !members.Contains(tu))) : !members.Contains(u));
        var outputs = region.Members.Where(Leaves).ToArray();
        if (outputs.Length == 0)
        {
            return; // dead code
        }

        var input = T.CreateBuffer((TensorType)region.Input.CheckedType, MemoryLocation.Input, out _, "x");
        var inside = new Dictionary<Expr, Expr>(ReferenceEqualityComparer.Instance) { [region.Input] = input };
        foreach (var call in region.Members)
        {
            var op = (IHipOp)call.Target;
            var arguments = call.Arguments.ToArray();
            for (int i = 0; i < op.Activations; i++)
            {
                arguments[i] = arguments[i] is IR.Tuple tuple
                    ? new IR.Tuple(tuple.Fields.ToArray().Select(f => inside[f]).ToArray())
                    : inside[arguments[i]];
            }

            inside[call] = new Call(call.Target, arguments); // constants (weights, bias, table) stay arguments and go to .rdata
        }

        var results = new TIR.Buffer[outputs.Length];
        var stores = new Expr[outputs.Length];
        for (int k = 0; k < outputs.Length; k++)
        {
            T.CreateBuffer((TensorType)outputs[k].CheckedType, MemoryLocation.Output, out results[k], $"y{k}");
            stores[k] = new Call(new HipStore(), inside[outputs[k]], results[k]);
        }

        var primFunction = new PrimFunction($"hip_{_count++}", HipRTModule.Kind, new Sequential(stores), new[] { input }.Concat(results).ToArray());
        var wrapper = new PrimFunctionWrapper(primFunction.Name + "_wrapper", primFunction, 1);
        CompilerServices.InferenceType(primFunction);
        module.Add(wrapper);
        module.Add(primFunction);

        var invocation = new Call(wrapper, region.Input);
        for (int k = 0; k < outputs.Length; k++)
        {
            Expr value = outputs.Length == 1 ? invocation : IR.F.Tensors.GetItem(invocation, k);
            CompilerServices.InferenceType(value);
            ReplaceUtility.ReplaceAllUsesWith(outputs[k], value);
        }
    }

    private sealed class Region
    {
        public Region(Expr input)
        {
            Input = input;
        }

        public Expr Input { get; }

        public List<Call> Members { get; } = new();

        public Region? MergedInto { get; set; }

        public Region Root => MergedInto is null ? this : MergedInto.Root;
    }

    // every hip call of a function body, producers before users
    private sealed class HipCalls : ExprWalker
    {
        private readonly List<Call> _calls;

        public HipCalls(List<Call> calls)
        {
            _calls = calls;
        }

        protected override Unit VisitLeafCall(Call expr)
        {
            if (IsHipCall(expr))
            {
                _calls.Add(expr);
            }

            return default;
        }
    }
}
