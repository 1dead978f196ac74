// Dequantize(a) -> MatMul(., Dequantize(B)) [-> Quantize]  ==>  HipQMatMul(a, B).
// The sub-graph of a QLinearMatMul import (src/Nncase.Importer/Onnx/QLinearMatmul.cs:25-28); without the
// trailing Quantize the product is written as float32 (one rounding of the exact integer sum).
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.PatternMatch;
using static Nncase.IR.TypePatternUtility;
using static Nncase.PatternMatch.F.Math;
using static Nncase.PatternMatch.Utility;

namespace Nncase.Passes.Rules.Hip;

[RuleGenerator]
public sealed partial class LowerMatMulToHip : IRewriteRule
{
    private static readonly Pattern Product = IsMatMul(
        "matmul",
        "product",
        _ => true,
        IsDequantize("dqLhs", null, _ => true, IsWildcard("lhs") with { TypePattern = HasFixedShape() & HasDataType(DataTypes.UInt8) }, IsTensorConst("lhsQp")),
        IsDequantize("dqRhs", null, _ => true, IsTensorConst("rhs", HasRank(2) & HasDataType(DataTypes.UInt8)), IsTensorConst("rhsQp")));

    public IPattern Pattern { get; } = IsAlt(
        IsQuantize("quantize", "output", q => q.TargetType == DataTypes.UInt8, Product, IsTensorConst("outputQp")),
        Product);

    private Expr? GetReplace(Expr lhs, TensorConst rhs, IMatchResult result, QuantParam lhsQp, QuantParam rhsQp)
    {
        bool requantised = result.GetValueOrDefault("outputQp") is TensorConst;
        var op = new HipQMatMul
        {
            LhsQuantParam = lhsQp,
            RhsQuantParam = rhsQp,
            OutputQuantParam = requantised ? ((TensorConst)result["outputQp"]).Value.ToScalar<QuantParam>() : new QuantParam(0, 1f),
            OutputType = requantised ? DataTypes.UInt8 : DataTypes.Float32,
        };
        return new Call(op, lhs, rhs);
    }
}
