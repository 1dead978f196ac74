// The operators of the hip module.  Activations are u8 NCHW tensors in the IR (the layout every nncase
// Conv2D has); the code generator records them as NHWC extents and the kernels run channels-last, so a hip
// function converts at its two ends only.
using System.Collections.Generic;
using System.Linq;
using Nncase.PatternMatch;
using static Nncase.IR.TypePatternUtility;

namespace Nncase.IR.Hip;

/// <summary>
/// u8 x u8 -> u8 / f32 convolution: y = Quantize(clamp(Conv2D(Dequantize(x), Dequantize(w)) + bias)).
/// Bias is int32 at scale xScale * wScale (Onnx/QLinearConv.cs:70).
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQConv2D : Op, IHipOp
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

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments)
    {
        var x = F.Math.Dequantize(arguments[0], InputQuantParam, DataTypes.Float32);
        var w = F.Math.Dequantize(arguments[1], WeightsQuantParam, DataTypes.Float32);
        var bias = F.Math.Dequantize(arguments[2], new QuantParam(0, InputQuantParam.Scale * WeightsQuantParam.Scale), DataTypes.Float32);
        var paddings = new[,] { { Paddings[0], Paddings[1] }, { Paddings[2], Paddings[3] } };
        Expr y = F.NN.Conv2D(x, w, bias, Strides, paddings, Dilations, PadMode.Constant, Groups, new[] { FusedClamp.Min, FusedClamp.Max });
        return OutputType == DataTypes.UInt8 ? F.Math.Quantize(y, OutputQuantParam, DataTypes.UInt8) : y;
    }
}

/// <summary>
/// u8 [M, K] x u8 [K, N] -> u8 / f32 product of a Dequantize -> MatMul (-> Quantize) chain; the right-hand side
/// is a constant (Onnx/QLinearMatmul.cs:25-28).
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQMatMul : Op, IHipOp
{
    public static readonly ParameterInfo Lhs = new(typeof(HipQMatMul), 0, "lhs", HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Rhs = new(typeof(HipQMatMul), 1, "rhs", HasRank(2) & HasDataType(DataTypes.UInt8));

    public QuantParam LhsQuantParam { get; init; }

    public QuantParam RhsQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public DataType OutputType { get; init; } = DataTypes.Float32;

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments)
    {
        Expr y = F.Math.MatMul(F.Math.Dequantize(arguments[0], LhsQuantParam, DataTypes.Float32), F.Math.Dequantize(arguments[1], RhsQuantParam, DataTypes.Float32));
        return OutputType == DataTypes.UInt8 ? F.Math.Quantize(y, OutputQuantParam, DataTypes.UInt8) : y;
    }
}

/// <summary>Implemented by every hip operator: the sub-graph of neutral operators it stands for.</summary>
public interface IHipOp
{
    /// <summary>Number of leading arguments that are activations (the rest are constants).</summary>
    int Activations { get; }

    /// <summary>
    /// Rebuilds the neutral sub-graph (Dequantize -> operator -> Quantize) over <paramref name="arguments"/>:
    /// what the lowering rule matched.  The evaluators of the operators without a device call of their own run
    /// it, and the outlining pass puts it back where an operator cannot join a hip function.
    /// </summary>
    Expr Raise(IReadOnlyList<Expr> arguments);
}

/// <summary>f32 -> u8 at the entry of a hip function: y = clamp(round(x / scale + zero_point), 0, 255).</summary>
[PatternFunctionalGenerator]
public sealed partial class HipQuantize : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipQuantize), 0, "input", HasRank(r => r == 2 || r == 4, "rank 2 or 4") & HasDataType(DataTypes.Float32));

    public QuantParam QuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments) => F.Math.Quantize(arguments[0], QuantParam, DataTypes.UInt8);
}

/// <summary>u8 -> f32 at the exit of a hip function: y = (x - zero_point) * scale.</summary>
[PatternFunctionalGenerator]
public sealed partial class HipDequantize : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipDequantize), 0, "input", HasRank(r => r == 2 || r == 4, "rank 2 or 4") & HasDataType(DataTypes.UInt8));

    public QuantParam QuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments) => F.Math.Dequantize(arguments[0], QuantParam, DataTypes.Float32);
}

/// <summary>u8 + u8 -> u8: y = Quantize(clamp(Dequantize(a) + Dequantize(b))), the residual add of a quantised network.</summary>
[PatternFunctionalGenerator]
public sealed partial class HipQAdd : Op, IHipOp
{
    public static readonly ParameterInfo Lhs = new(typeof(HipQAdd), 0, "lhs", HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Rhs = new(typeof(HipQAdd), 1, "rhs", HasDataType(DataTypes.UInt8));

    public QuantParam LhsQuantParam { get; init; }

    public QuantParam RhsQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public ValueRange<float> FusedClamp { get; init; } = ValueRange<float>.Full;

    public int Activations => 2;

    public Expr Raise(IReadOnlyList<Expr> arguments)
    {
        Expr sum = F.Math.Binary(BinaryOp.Add, F.Math.Dequantize(arguments[0], LhsQuantParam, DataTypes.Float32), F.Math.Dequantize(arguments[1], RhsQuantParam, DataTypes.Float32));
        if (!(float.IsNegativeInfinity(FusedClamp.Min) && float.IsPositiveInfinity(FusedClamp.Max)))
        {
            sum = F.Math.Clamp(sum, FusedClamp.Min, FusedClamp.Max);
        }

        return F.Math.Quantize(sum, OutputQuantParam, DataTypes.UInt8);
    }
}

/// <summary>u8 [N, C, H, W] -> u8 [N, C, 1, 1]: the mean over H and W between Dequantize and Quantize.</summary>
[PatternFunctionalGenerator]
public sealed partial class HipQGlobalAvgPool : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipQGlobalAvgPool), 0, "input", HasRank(4) & HasDataType(DataTypes.UInt8));

    public QuantParam InputQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments) =>
        F.Math.Quantize(F.Tensors.ReduceMean(F.Math.Dequantize(arguments[0], InputQuantParam, DataTypes.Float32), new[] { 2, 3 }, 0f, true), OutputQuantParam, DataTypes.UInt8);
}

/// <summary>
/// u8 -> u8 through a table of 256 bytes: any per-element function between Dequantize and Quantize (swish,
/// sigmoid, leaky relu, a Unary).  The lowering rule fills the table by running the matched sub-graph over the
/// 256 byte values with the compiler's own evaluator, so the table holds the bytes the float path gives.
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQLut : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipQLut), 0, "input", HasDataType(DataTypes.UInt8));

    public static readonly ParameterInfo Table = new(typeof(HipQLut), 1, "table", HasShape(new Shape(256)) & HasDataType(DataTypes.UInt8));

    public QuantParam InputQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public int Activations => 1;

    // Gather(table, axis 0, x) is the table applied element by element
    public Expr Raise(IReadOnlyList<Expr> arguments) =>
        F.Tensors.Gather(arguments[1], 0, F.Tensors.Cast(arguments[0], DataTypes.Int64));
}

/// <summary>
/// Channel concatenation of u8 tensors, each with its own QuantParam, requantised to the output's:
/// y = Quantize(Concat(Dequantize(x_0), ..., axis 1)).  Takes the tensors as one tuple, like Concat.
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQConcat : Op, IHipOp
{
    public static readonly ParameterInfo Inputs = new(typeof(HipQConcat), 0, "inputs", IsTuple());

    public IRArray<QuantParam> InputQuantParams { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments)
    {
        var fields = ((IR.Tuple)arguments[0]).Fields.ToArray();
        var floats = fields.Select((x, i) => (Expr)F.Math.Dequantize(x, InputQuantParams[i], DataTypes.Float32)).ToArray();
        return F.Math.Quantize(F.Tensors.Concat(new IR.Tuple(floats), 1), OutputQuantParam, DataTypes.UInt8);
    }
}

/// <summary>Nearest-neighbour resize of a u8 [N, C, H, W] tensor to [N, C, OutH, OutW]; bytes are copied, so the QuantParam is the input's.</summary>
[PatternFunctionalGenerator]
public sealed partial class HipResizeNearest : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipResizeNearest), 0, "input", HasRank(4) & HasDataType(DataTypes.UInt8));

    public int OutH { get; init; }

    public int OutW { get; init; }

    public ImageResizeTransformationMode TransformationMode { get; init; } = ImageResizeTransformationMode.Asymmetric;

    public ImageResizeNearestMode NearestMode { get; init; } = ImageResizeNearestMode.Floor;

    public QuantParam QuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments)
    {
        var shape = arguments[0].CheckedShape.ToValueArray();
        return F.Imaging.ResizeImage(ImageResizeMode.NearestNeighbor, TransformationMode, NearestMode, arguments[0], None.Default, new[] { shape[0], shape[1], OutH, OutW }, None.Default, None.Default, None.Default);
    }
}

/// <summary>
/// Square max pooling of a u8 tensor between Dequantize and Quantize (ReduceWindow2D with ReduceOp.Max, the
/// same padding on all four sides, dilation 1, floor mode).
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipQMaxPool : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipQMaxPool), 0, "input", HasRank(4) & HasDataType(DataTypes.UInt8));

    public int Kernel { get; init; }

    public int Stride { get; init; }

    public int Padding { get; init; }

    public float InitValue { get; init; } = float.NegativeInfinity;

    public QuantParam InputQuantParam { get; init; }

    public QuantParam OutputQuantParam { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments) =>
        F.Math.Quantize(
            F.NN.ReduceWindow2D(ReduceOp.Max, F.Math.Dequantize(arguments[0], InputQuantParam, DataTypes.Float32), InitValue, new[] { Kernel, Kernel }, new[] { Stride, Stride }, new[,] { { Padding, Padding }, { Padding, Padding } }, new[] { 1, 1 }, false, false),
            OutputQuantParam,
            DataTypes.UInt8);
}

/// <summary>
/// [N, C, 1, 1] <-> [N, C] of a u8 tensor between hip operators (the Reshape between a global mean and the
/// classifier's matrix product): the bytes stay where they are.
/// </summary>
[PatternFunctionalGenerator]
public sealed partial class HipReshape : Op, IHipOp
{
    public static readonly ParameterInfo Input = new(typeof(HipReshape), 0, "input", HasDataType(DataTypes.UInt8));

    public IRArray<int> NewShape { get; init; }

    public int Activations => 1;

    public Expr Raise(IReadOnlyList<Expr> arguments) => F.Tensors.Reshape(arguments[0], NewShape.ToArray());
}

/// <summary>
/// The statement of a hip PrimFunction's body: the function writes <c>value</c> to its output buffer
/// <c>destination</c>.  One per output, in parameter order.
/// </summary>
public sealed partial class HipStore : Op
{
    public static readonly ParameterInfo Value = new(typeof(HipStore), 0, "value");

    public static readonly ParameterInfo Destination = new(typeof(HipStore), 1, "destination");

    public override bool CanFoldConstCall => false;
}
