// Dequantize(x) -> Conv2D(., Dequantize(W), bias) -> Quantize  ==>  HipQConv2D(x, W, int32 bias).
// The sub-graph is what the ONNX and TFLite importers emit for a quantised convolution
// (src/Nncase.Importer/Onnx/QLinearConv.cs:61-75, TFLite/Conv2D.cs:39-98) and what the quantiser leaves after
// PTQ; the K210 target lowers its convolutions at the same place
// (modules/Nncase.Modules.K210/Transform/Rules/K210/LowerConv2D.cs:43-93).
using System;
using System.Linq;
using Nncase.IR;
using Nncase.IR.Hip;
using Nncase.IR.Math;
using Nncase.PatternMatch;
using static Nncase.IR.TypePatternUtility;
using static Nncase.PatternMatch.F.Math;
using static Nncase.PatternMatch.F.NN;
using static Nncase.PatternMatch.Utility;

namespace Nncase.Passes.Rules.Hip;

[RuleGenerator]
public sealed partial class LowerConv2DToHip : IRewriteRule
{
    public IPattern Pattern { get; } = IsQuantize(
        "quantize",
        "output",
        q => q.TargetType == DataTypes.UInt8,
        IsConv2D(
            "conv",
            "convCall",
            c => c.PadMode == PadMode.Constant,
            IsDequantize("dqInput", null, _ => true, IsWildcard("input") with { TypePattern = HasFixedShape() & HasDataType(DataTypes.UInt8) }, IsTensorConst("inputQp")),
            IsDequantize("dqWeights", null, _ => true, IsTensorConst("weights", HasDataType(DataTypes.UInt8)), IsTensorConst("weightsQp")),
            IsAlt(
                IsDequantize("dqBias", null, _ => true, IsTensorConst("bias", HasDataType(DataTypes.Int32)), IsTensorConst("biasQp")),
                IsTensorConst("zeroBias")),
            IsTensorConst("strides"),
            IsTensorConst("paddings"),
            IsTensorConst("dilations"),
            IsTensorConst("groups"),
            IsTensorConst("fusedClamp")),
        IsTensorConst("outputQp"));

    private Expr? GetReplace(Expr input, TensorConst weights, IMatchResult result, QuantParam inputQp, QuantParam weightsQp, QuantParam outputQp, int[] strides, Tensor<int> paddings, int[] dilations, int groups, float[] fusedClamp)
    {
        int outChannels = weights.CheckedShape[0].FixedValue;
        int[] biasValues;
        if (result.GetValueOrDefault("bias") is TensorConst bias)
        {
            // the importer gives the bias at scale xScale * wScale (one float product, Onnx/QLinearConv.cs:70) with zero
            // point 0: those integers are the accumulator's own units; any other scale, however close, would need a
            // rescale and stays on the float path
            var biasQp = ((TensorConst)result["biasQp"]).Value.ToScalar<QuantParam>();
            if (biasQp.ZeroPoint != 0 || biasQp.Scale != inputQp.Scale * weightsQp.Scale)
            {
                return null;
            }

            biasValues = bias.Value.ToArray<int>();
        }
        else
        {
            var zero = ((TensorConst)result["zeroBias"]).Value.ToArray<float>();
            if (zero.Any(v => v != 0f))
            {
                return null;
            }

            biasValues = new int[outChannels];
        }

        var op = new HipQConv2D
        {
            Strides = strides,
            Dilations = dilations,
            Paddings = new[] { paddings[0, 0], paddings[0, 1], paddings[1, 0], paddings[1, 1] },
            Groups = groups,
            InputQuantParam = inputQp,
            WeightsQuantParam = weightsQp,
            OutputQuantParam = outputQp,
            FusedClamp = new ValueRange<float>(fusedClamp[0], fusedClamp[1]),
            OutputType = DataTypes.UInt8,
        };
        return new Call(op, input, weights, Tensor.From(biasValues));
    }
}
