// The two operators of the hip module.  Activations are u8 NCHW tensors in the IR (the layout every nncase
// Conv2D has); the code generator records them as NHWC extents and the kernels run channels-last, so a hip
// function converts at its two ends only.
using Nncase.PatternMatch;
using static Nncase.IR.TypePatternUtility;

namespace Nncase.IR.Hip;

/// <summary>
/// u8 x u8 -> u8 / f32 convolution: y = Quantize(clamp(Conv2D(Dequantize(x), Dequantize(w)) + bias)).
/// Bias is int32 at scale xScale * wScale (Onnx/QLinearConv.cs:70).
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQConv2D : Op
{
    public static readonly ParameterInfo Input = new(typeof(HipQConv2D), 0, "input", HasRank(4) & HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Weights = new(typeof(HipQConv2D), 1, "weights", HasRank(4) & HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Bias = new(typeof(HipQConv2D), 2, "bias", HasRank(1) & HasDataType(DataTypes.Int32));

    public int[] Strides { get; init; } = { 1, 1 };

    public int[] Dilations { get; init; } = { 1, 1 };

    /// <summary>Gets top, bottom, left, right.</summary>
    public int[] Paddings { get; init; } = { 0, 0, 0, 0 };

    public int Groups { get; init; } = 1;

    public QuantParam InputQuantParam { get; init; }

    public QuantParam WeightsQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public ValueRange<float> FusedClamp { get; init; } = ValueRange<float>.Full;

    /// <summary>Gets UInt8 (requantised) or Float32 (the Quantize consumer is absent).</summary>
    public DataType OutputType { get; init; } = DataTypes.UInt8;
}

/// <summary>
/// u8 [M, K] x u8 [K, N] -> u8 / f32 product of a Dequantize -> MatMul (-> Quantize) chain; the right-hand side
/// is a constant (Onnx/QLinearMatmul.cs:25-28).
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQMatMul : Op
{
    public static readonly ParameterInfo Lhs = new(typeof(HipQMatMul), 0, "lhs", HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Rhs = new(typeof(HipQMatMul), 1, "rhs", HasRank(2) & HasDataType(DataTypes.UInt8));

    public QuantParam LhsQuantParam { get; init; }

    public QuantParam RhsQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public DataType OutputType { get; init; } = DataTypes.Float32;
}
