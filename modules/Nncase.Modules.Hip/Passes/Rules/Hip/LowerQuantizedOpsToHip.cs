// Lowering rules for the operators of a quantised network other than its convolutions and matrix products.
// After PTQ (or in a QDQ import) each of them sits between Dequantize and Quantize calls with constant
// QuantParams; a rule replaces that sandwich by one hip operator on the u8 tensors.  The K210 target lowers its
// own operators at the same place and in the same style
// (modules/Nncase.Modules.K210/Transform/Rules/K210/LowerConv2D.cs:43-93).
//
// The rules of this file run in the "lowering_hip" pass together with the convolution and matmul rules.  The
// two boundary rules at the end (a lone Quantize / Dequantize next to a hip operator) run in a pass of their
// own afterwards, because every sandwich rule needs the Dequantize calls still in place.
using System;
using System.Collections.Generic;
using System.Linq;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.IR.Imaging;
using Nncase.IR.Math;
using Nncase.IR.NN;
using Nncase.IR.Tensors;
using Nncase.PatternMatch;
using static Nncase.IR.TypePatternUtility;
using static Nncase.PatternMatch.F.Imaging;
using static Nncase.PatternMatch.F.Math;
using static Nncase.PatternMatch.F.NN;
using static Nncase.PatternMatch.F.Tensors;
using static Nncase.PatternMatch.Utility;

namespace Nncase.Passes.Rules.Hip;

internal static class HipPatterns
{
    /// <summary>Dequantize(u8 tensor of fixed shape, constant QuantParam) with the given capture names.</summary>
    public static Pattern DequantizedInput(string input, string quantParam) =>
        IsDequantize(_ => true, IsWildcard(input) with { TypePattern = HasFixedShape() & HasDataType(DataTypes.UInt8) }, IsTensorConst(quantParam));

    public static QuantParam QuantParamOf(Expr constant) => ((TensorConst)constant).Value.ToScalar<QuantParam>();

    public static bool IsHipCall(Expr expr) => expr is Call { Target: IHipOp };
}

/// <summary>Quantize(Clamp?(Dequantize(a) + Dequantize(b))) ==> HipQAdd(a, b): the residual add.</summary>
[RuleGenerator]
public sealed partial class LowerAddToHip : IRewriteRule
{
    private static readonly Pattern Sum = IsBinary(
        "add",
        "addCall",
        b => b.BinaryOp == BinaryOp.Add,
        HipPatterns.DequantizedInput("lhs", "lhsQp"),
        HipPatterns.DequantizedInput("rhs", "rhsQp"));

    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsAlt(IsClamp(Sum, IsTensorConst("min", IsFloatScalar()), IsTensorConst("max", IsFloatScalar())), Sum),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(Expr lhs, Expr rhs, QuantParam lhsQp, QuantParam rhsQp, QuantParam outputQp, IMatchResult result)
    {
        // the device adds element by element: no broadcasting
        if (!lhs.CheckedShape.ToValueArray().SequenceEqual(rhs.CheckedShape.ToValueArray()))
        {
            return null;
        }

        var clamp = ValueRange<float>.Full;
        if (result.GetValueOrDefault("min") is TensorConst min)
        {
            clamp = new ValueRange<float>(min.Value.ToScalar<float>(), ((TensorConst)result["max"]).Value.ToScalar<float>());
        }

        return new Call(new HipQAdd { LhsQuantParam = lhsQp, RhsQuantParam = rhsQp, OutputQuantParam = outputQp, FusedClamp = clamp }, lhs, rhs);
    }
}

/// <summary>Quantize(ReduceMean(Dequantize(x), axes {2, 3}, keepDims)) ==> HipQGlobalAvgPool(x).</summary>
[RuleGenerator]
public sealed partial class LowerReduceMeanToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsReduce(
            "reduce",
            "reduceCall",
            r => r.ReduceOp == ReduceOp.Mean,
            HipPatterns.DequantizedInput("input", "inputQp"),
            IsTensorConst("axes"),
            IsTensorConst("initValue"),
            IsTensorConst("keepDims")),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(Expr input, QuantParam inputQp, QuantParam outputQp, int[] axes, TensorConst keepDims)
    {
        var spatial = axes.Select(a => a < 0 ? a + 4 : a).OrderBy(a => a).ToArray();
        if (input.CheckedShape.Rank != 4 || keepDims.Value.ToScalar<int>() == 0 || !spatial.SequenceEqual(new[] { 2, 3 }))
        {
            return null;
        }

        return new Call(new HipQGlobalAvgPool { InputQuantParam = inputQp, OutputQuantParam = outputQp }, input);
    }
}

/// <summary>
/// Quantize(ReduceWindow2D(Mean / Max, Dequantize(x), ...)) ==> HipQGlobalAvgPool(x) when the mean window is the
/// whole image, HipQMaxPool(x) for a square max window with one padding on all sides.
/// </summary>
[RuleGenerator]
public sealed partial class LowerReduceWindow2DToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsReduceWindow2D(
            "pool",
            "poolCall",
            p => p.ReduceOp is ReduceOp.Mean or ReduceOp.Max,
            HipPatterns.DequantizedInput("input", "inputQp"),
            IsTensorConst("initValue"),
            IsTensorConst("filter"),
            IsTensorConst("stride"),
            IsTensorConst("padding"),
            IsTensorConst("dilation"),
            IsTensorConst("ceilMode"),
            IsTensorConst("countIncludePad")),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(ReduceWindow2D pool, Expr input, QuantParam inputQp, QuantParam outputQp, float initValue, int[] filter, int[] stride, Tensor<int> padding, int[] dilation, bool ceilMode)
    {
        var shape = input.CheckedShape.ToValueArray();
        int[] pads = { padding[0, 0], padding[0, 1], padding[1, 0], padding[1, 1] };
        if (dilation[0] != 1 || dilation[1] != 1 || ceilMode)
        {
            return null;
        }

        if (pool.ReduceOp == ReduceOp.Mean)
        {
            // one window over the whole image: a global mean, whatever the stride says
            bool global = filter[0] == shape[2] && filter[1] == shape[3] && pads.All(p => p == 0);
            return global ? new Call(new HipQGlobalAvgPool { InputQuantParam = inputQp, OutputQuantParam = outputQp }, input) : null;
        }

        // the device starts the maximum at code 0, so the initial value must not exceed what code 0 stands for
        float lowest = (0 - inputQp.ZeroPoint) * inputQp.Scale;
        if (filter[0] != filter[1] || stride[0] != stride[1] || pads.Any(p => p != pads[0]) || !(initValue <= lowest))
        {
            return null;
        }

        return new Call(new HipQMaxPool { Kernel = filter[0], Stride = stride[0], Padding = pads[0], InitValue = initValue, InputQuantParam = inputQp, OutputQuantParam = outputQp }, input);
    }
}

/// <summary>
/// Quantize(f(Dequantize(x))) for a per-element f (an activation with scalar parameters, or a Unary)
/// ==> HipQLut(x, table), table[v] = the byte the matched sub-graph gives for the byte v.
/// </summary>
[RuleGenerator]
public sealed partial class LowerActivationToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsAlt(
            IsCall("actCall", IsOp<ActivationOp>("activation", _ => true), IsVArgsRepeat("parameters", inputs =>
            {
                var patterns = new Pattern[inputs.Length];
                patterns[0] = HipPatterns.DequantizedInput("input", "inputQp");
                for (int i = 1; i < inputs.Length; i++)
                {
                    patterns[i] = IsTensorConst(null, IsScalar());
                }

                return patterns;
            })),
            IsUnary("unary", "unaryCall", _ => true, HipPatterns.DequantizedInput("input", "inputQp"))),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(Expr input, QuantParam inputQp, QuantParam outputQp, IMatchResult result)
    {
        var codes = Tensor.From(Enumerable.Range(0, 256).Select(v => (byte)v).ToArray(), new[] { 256 });
        Expr x = IR.F.Math.Dequantize(codes, inputQp, DataTypes.Float32);
        Expr y;
        if (result.GetValueOrDefault("actCall") is Call actCall)
        {
            y = new Call(actCall.Target, new[] { x }.Concat(actCall.Arguments.ToArray().Skip(1)).ToArray());
        }
        else
        {
            y = new Call(((Call)result["unaryCall"]).Target, x);
        }

        // the compiler's evaluator runs the reference kernels: these are the bytes the float path produces
        var table = IR.F.Math.Quantize(y, outputQp, DataTypes.UInt8).Evaluate().AsTensor();
        return new Call(new HipQLut { InputQuantParam = inputQp, OutputQuantParam = outputQp }, input, table);
    }
}

/// <summary>Quantize(Concat((Dequantize(x_0), ...), axis 1)) ==> HipQConcat((x_0, ...)).</summary>
[RuleGenerator]
public sealed partial class LowerConcatToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsConcat(
            "concat",
            "concatCall",
            _ => true,
            PatternMatch.Utility.IsTuple(null, IsVArgsRepeat("tupleInputs", fields =>
            {
                var patterns = new Pattern[fields.Length];
                for (int i = 0; i < patterns.Length; i++)
                {
                    patterns[i] = HipPatterns.DequantizedInput($"input_{i}", $"inputQp_{i}");
                }

                return patterns;
            }))),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(Concat concat, IReadOnlyList<Expr> tupleInputs, QuantParam outputQp, IMatchResult result)
    {
        var inputs = Enumerable.Range(0, tupleInputs.Count).Select(i => (Expr)result[$"input_{i}"]).ToArray();
        var qps = Enumerable.Range(0, tupleInputs.Count).Select(i => HipPatterns.QuantParamOf((Expr)result[$"inputQp_{i}"])).ToArray();
        return HipConcat.Build(concat.Axis, inputs, qps, outputQp);
    }
}

/// <summary>
/// Concat((x_0, ...), axis 1) of u8 tensors ==> HipQConcat with one QuantParam for all: the form the quantiser
/// leaves once CombineQuantizeConcat (src/Nncase.Passes/Rules/Neutral/CombineQuantize.cs:30-80) has moved the
/// Quantize calls onto the inputs.  Bytes are copied.
/// </summary>
[RuleGenerator]
public sealed partial class LowerByteConcatToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsConcat(
        "concat",
        "concatCall",
        _ => true,
        PatternMatch.Utility.IsTuple(null, IsVArgsRepeat("tupleInputs", () => IsWildcard() with { TypePattern = HasFixedShape() & HasDataType(DataTypes.UInt8) })));

    private Expr? GetReplace(Concat concat, IReadOnlyList<Expr> tupleInputs)
    {
        // only inside a hip region: a byte concat between stackvm operators gains nothing from the device
        if (!tupleInputs.Any(HipPatterns.IsHipCall))
        {
            return null;
        }

        var same = new QuantParam(0, 1f);
        return HipConcat.Build(concat.Axis, tupleInputs.ToArray(), tupleInputs.Select(_ => same).ToArray(), same);
    }
}

internal static class HipConcat
{
    public const int MaxInputs = 8; // the operator record of a hip function holds eight tensor indices

    public static Expr? Build(int axis, Expr[] inputs, QuantParam[] qps, QuantParam outputQp)
    {
        int rank = inputs[0].CheckedShape.Rank;
        if (rank != 4 || (axis < 0 ? axis + rank : axis) != 1 || inputs.Length > MaxInputs)
        {
            return null;
        }

        return new Call(new HipQConcat { InputQuantParams = qps, OutputQuantParam = outputQp }, new IR.Tuple(inputs));
    }
}

/// <summary>
/// Nearest-neighbour ResizeImage of a u8 tensor, directly or as Quantize(ResizeImage(Dequantize(x))) with the
/// same QuantParam on both sides ==> HipResizeNearest(x).
/// </summary>
[RuleGenerator]
public sealed partial class LowerResizeToHip : IRewriteRule
{
    private static Pattern Resize(Pattern input) => IsResizeImage(
        "resize",
        "resizeCall",
        r => r.ResizeMode == ImageResizeMode.NearestNeighbor && !r.IsTFResize && r.TransformationMode != ImageResizeTransformationMode.TFCropAndResize,
        input,
        IsWildcard("roi"),
        IsTensorConst("newSize"),
        IsWildcard("cubicCoeffA"),
        IsWildcard("excludeOutside"),
        IsWildcard("extrapolationValue"));

    public IPattern Pattern { get; } = IsAlt(
        IsQuantize("quantize", "output", q => q.TargetType == DataTypes.UInt8, Resize(HipPatterns.DequantizedInput("input", "inputQp")), IsTensorConst("outputQp")),
        Resize(IsWildcard("input") with { TypePattern = HasFixedShape() & HasRank(4) & HasDataType(DataTypes.UInt8) }));

    private Expr? GetReplace(ResizeImage resize, Expr input, int[] newSize, IMatchResult result)
    {
        var qp = new QuantParam(0, 1f);
        if (result.GetValueOrDefault("outputQp") is TensorConst outputQp)
        {
            qp = HipPatterns.QuantParamOf(outputQp);
            var inputQp = HipPatterns.QuantParamOf((Expr)result["inputQp"]);
            if (inputQp.ZeroPoint != qp.ZeroPoint || inputQp.Scale != qp.Scale)
            {
                return null; // a requantising resize stays on the float path
            }
        }
        else if (!HipPatterns.IsHipCall(input))
        {
            return null; // a byte resize between stackvm operators stays where it is
        }

        var shape = input.CheckedShape.ToValueArray();
        if (shape.Length != 4 || newSize.Length != 4 || newSize[0] != shape[0] || newSize[1] != shape[1])
        {
            return null;
        }

        return new Call(new HipResizeNearest { OutH = newSize[2], OutW = newSize[3], TransformationMode = resize.TransformationMode, NearestMode = resize.NearestMode, QuantParam = qp }, input);
    }
}

/// <summary>Quantize(f32 x) whose users are all hip operators ==> HipQuantize(x): the entry of a hip function.</summary>
[RuleGenerator]
public sealed partial class LowerQuantizeToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsWildcard("input") with { TypePattern = HasFixedShape() & HasRank(r => r == 2 || r == 4, "rank 2 or 4") & HasDataType(DataTypes.Float32) },
        IsTensorConst("quantParam"));

    private Expr? GetReplace(Call output, Expr input, QuantParam quantParam)
    {
        // (a tuple of a HipQConcat stands between the value and the operator that reads it)
        bool feedsHip = output.Users.Count > 0 && output.Users.All(u => HipPatterns.IsHipCall(u) || (u is IR.Tuple t && t.Users.All(HipPatterns.IsHipCall)));
        return feedsHip && input is not Const ? new Call(new HipQuantize { QuantParam = quantParam }, input) : null;
    }
}

/// <summary>Dequantize(value of a hip operator) ==> HipDequantize: the exit of a hip function.</summary>
[RuleGenerator]
public sealed partial class LowerDequantizeToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsDequantize(
        "dequantize",
        "output",
        d => d.TargetType == DataTypes.Float32,
        IsWildcard("input") with { TypePattern = HasFixedShape() & HasRank(r => r == 2 || r == 4, "rank 2 or 4") & HasDataType(DataTypes.UInt8) },
        IsTensorConst("quantParam"));

    private Expr? GetReplace(Expr input, QuantParam quantParam) =>
        HipPatterns.IsHipCall(input) ? new Call(new HipDequantize { QuantParam = quantParam }, input) : null;
}

/// <summary>Reshape([N, C, 1, 1] -> [N, C]) or back, of the value of a hip operator ==> HipReshape.</summary>
[RuleGenerator]
public sealed partial class LowerReshapeToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsReshape(
        "reshape",
        "output",
        _ => true,
        IsWildcard("input") with { TypePattern = HasFixedShape() & HasDataType(DataTypes.UInt8) },
        IsTensorConst("newShape"));

    private Expr? GetReplace(Call output, Expr input)
    {
        if (!HipPatterns.IsHipCall(input) || !output.CheckedShape.IsFixed)
        {
            return null;
        }

        // (-1 entries of the constant are resolved in the call's checked shape)
        int[] from = input.CheckedShape.ToValueArray(), to = output.CheckedShape.ToValueArray();
        static bool Flat(int[] four, int[] two) => four.Length == 4 && two.Length == 2 && four[2] == 1 && four[3] == 1 && four[0] == two[0] && four[1] == two[1];
        return Flat(from, to) || Flat(to, from) ? new Call(new HipReshape { NewShape = to }, input) : null;
    }
}
