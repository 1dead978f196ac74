// Evaluators of the hip operators that have no device call in the compiler: each one evaluates the neutral
// sub-graph it stands for (IHipOp.Raise) with the compiler's own kernels.  The device kernels give the same
// bytes (their tests compare them with a restatement of those kernels), so calibration, constant folding and
// dumped per-layer results agree with what the kmodel produces.  Type and cost come from the same sub-graph.
using System;
using System.Collections.Generic;
using System.Linq;
using Nncase.CostModel;
using Nncase.IR;
using Nncase.IR.Hip;

namespace Nncase.Evaluator.Hip;

public abstract class HipRaisedEvaluator<T> : IEvaluator<T>, ITypeInferencer<T>, ICostEvaluator<T>
    where T : Op, IHipOp
{
    public IValue Visit(IEvaluateContext context, T target)
    {
        var arguments = target.Parameters.Select(p => AsExpr(context.GetArgumentValue(target, p))).ToArray();
        return target.Raise(arguments).Evaluate();
    }

    public IRType Visit(ITypeInferenceContext context, T target)
    {
        // constants (a table, weights) keep their values: Raise may read them
        var arguments = target.Parameters.Select((p, i) => i < target.Activations ? Placeholder(context.GetArgumentType(target, p)) : context.GetArgument(target, p)).ToArray();
        if (arguments.Any(a => a is null))
        {
            return new InvalidType("hip operators take tensors, or one tuple of tensors");
        }

        var raised = target.Raise(arguments!);
        return CompilerServices.InferenceType(raised) ? raised.CheckedType : new InvalidType($"{typeof(T).Name}: the operators it stands for do not accept these arguments");
    }

    public Cost Visit(ICostEvaluateContext context, T target)
    {
        // one pass over the operands and the result: these operators move bytes
        var output = context.GetReturnType<IRType>();
        var cost = new Cost { [CostFactorNames.MemoryStore] = CostUtility.GetMemoryAccess(output) };
        UInt128 load = 0;
        foreach (var p in target.Parameters)
        {
            load += CostUtility.GetMemoryAccess(context.GetArgumentType<IRType>(target, p));
        }

        cost[CostFactorNames.MemoryLoad] = load;
        return cost;
    }

    private static Expr AsExpr(IValue value) => value switch
    {
        TensorValue t => Const.FromTensor(t.AsTensor()),
        TupleValue tuple => new IR.Tuple(tuple.AsTensors().Select(t => (Expr)Const.FromTensor(t)).ToArray()),
        _ => throw new NotSupportedException($"{value.GetType().Name} as the argument of a hip operator"),
    };

    private static Expr? Placeholder(IRType type) => type switch
    {
        TensorType t => new Var(t),
        TupleType tuple when tuple.All(f => f is TensorType) => new IR.Tuple(tuple.Select(f => (Expr)new Var(f)).ToArray()),
        _ => null,
    };
}

public sealed class HipQuantizeEvaluator : HipRaisedEvaluator<HipQuantize>
{
}

public sealed class HipDequantizeEvaluator : HipRaisedEvaluator<HipDequantize>
{
}

public sealed class HipQAddEvaluator : HipRaisedEvaluator<HipQAdd>
{
}

public sealed class HipQGlobalAvgPoolEvaluator : HipRaisedEvaluator<HipQGlobalAvgPool>
{
}

public sealed class HipQLutEvaluator : HipRaisedEvaluator<HipQLut>
{
}

public sealed class HipQConcatEvaluator : HipRaisedEvaluator<HipQConcat>
{
}

public sealed class HipResizeNearestEvaluator : HipRaisedEvaluator<HipResizeNearest>
{
}

public sealed class HipQMaxPoolEvaluator : HipRaisedEvaluator<HipQMaxPool>
{
}

public sealed class HipReshapeEvaluator : HipRaisedEvaluator<HipReshape>
{
}

/// <summary>HipStore is a statement: it has no value.</summary>
public sealed class HipStoreEvaluator : ITypeInferencer<HipStore>
{
    public IRType Visit(ITypeInferenceContext context, HipStore target)
    {
        var value = context.GetArgumentType(target, HipStore.Value);
        var destination = context.GetArgumentType(target, HipStore.Destination);
        return value is TensorType v && destination is TensorType d && v.Equals(d)
            ? TupleType.Void
            : new InvalidType("HipStore writes a tensor to a buffer of its type");
    }
}
