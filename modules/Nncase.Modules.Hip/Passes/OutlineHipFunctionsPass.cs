// Moves every maximal chain of hip operators out of the stackvm functions into a function of module kind
// "hip", so that the kmodel gets a hip module whose functions the stackvm code reaches through EXTCALL
// (src/Native/src/runtime/stackvm/ops/control.cpp:25-75).
//
// A chain starts at a hip call whose activation does not come from another hip call, and grows while the
// value has exactly one user and that user is a hip call taking it as its activation.  The chain becomes
//   Fusion("hip_<n>", "hip", body, x)            (src/Nncase.Core/IR/Fusion.cs:21-23)
// added to the module (ModelBuilder groups functions by ModuleKind, src/Nncase.CodeGen/CodeGen/ModelBuilder.cs:33-45)
// and the call site becomes Call(fusion, x).  The stackvm code generator emits that call as
// "LdFunctionId ; EXTCALL args, false" once its VisitLeafCall accepts a Fusion of another module kind beside
// Function (modules/Nncase.Modules.StackVM/CodeGen/StackVM/CodegenVisitor.cs:306-310).
using System.Collections.Generic;
using System.Linq;
using System.Threading.Tasks;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.Runtime.Hip;

namespace Nncase.Passes;

public sealed class OutlineHipFunctionsPass : ModulePass
{
    private int _count;

    protected override Task<IRModule> RunCoreAsync(IRModule module, RunPassContext context)
    {
        foreach (var function in module.Functions.OfType<Function>().ToArray())
        {
            var tails = new List<Call>();
            new ChainTails(tails).Visit(function.Body);
            foreach (var tail in tails)
            {
                Outline(module, tail);
            }
        }

        return Task.FromResult(module);
    }

    private static bool IsHipCall(Expr expr) => expr is Call { Target: HipQConv2D or HipQMatMul };

    private static Expr Activation(Call call) => call.Arguments[0];

    // `call` continues a chain when it is the only user of a hip call's value, as that call's activation
    private static bool ContinuesChain(Call call) =>
        IsHipCall(Activation(call)) && Activation(call).Users.Count == 1;

    private void Outline(IRModule module, Call tail)
    {
        var chain = new List<Call> { tail };
        while (ContinuesChain(chain[^1]))
        {
            chain.Add((Call)Activation(chain[^1]));
        }

        chain.Reverse(); // head first
        var external = Activation(chain[0]);
        var parameter = new Var("x", external.CheckedType);
        Expr body = parameter;
        foreach (var call in chain)
        {
            var arguments = call.Arguments.ToArray();
            arguments[0] = body; // constants (weights, bias) stay arguments of the call and go to .rdata
            body = new Call(call.Target, arguments);
        }

        var fusion = new Fusion($"hip_{_count++}", HipRTModule.Kind, body, parameter);
        module.Add(fusion);
        var replacement = new Call(fusion, external);
        IRHelpers.ReplaceAllUsesWith(tail, replacement);
    }

    // collects the last call of every chain, in post order
    private sealed class ChainTails : ExprWalker
    {
        private readonly List<Call> _tails;

        public ChainTails(List<Call> tails)
        {
            _tails = tails;
        }

        protected override Unit VisitLeafCall(Call expr)
        {
            if (IsHipCall(expr))
            {
                bool extended = expr.Users.Count == 1 && expr.Users.First() is Call user && IsHipCall(user) && ReferenceEquals(Activation(user), expr);
                if (!extended)
                {
                    _tails.Add(expr);
                }
            }

            return default;
        }
    }
}
